"""Pins the CPU oracle against things it did not compute itself: the reference's
known answers, torch-CPU library routines, exact rational arithmetic on small
inputs, and invariants of the domain.  No GPU."""
from fractions import Fraction

import numpy as np
import pytest
import torch

from oracle import oracle as O


# ---------------------------------------------------------------- helpers
def _frac_of_bf16(bits: int) -> Fraction:
    sign = -1 if bits >> 15 else 1
    e = (bits >> 7) & 0xFF
    m = bits & 0x7F
    assert e != 0xFF
    if e == 0:
        return sign * Fraction(m, 1 << 7) * Fraction(2) ** (-126)
    return sign * (1 + Fraction(m, 1 << 7)) * Fraction(2) ** (e - 127)


def _round_frac(x: Fraction, p: int, emin: int) -> Fraction:
    """Round an exact rational to a binary float with p significand bits (RNE),
    gradual underflow at exponent emin.  Independent restatement of IEEE
    rounding used to brute-force the oracle."""
    if x == 0:
        return Fraction(0)
    s = -1 if x < 0 else 1
    a = abs(x)
    e = 0
    while a >= 2:
        a /= 2; e += 1
    while a < 1:
        a *= 2; e -= 1
    e = max(e, emin)
    ulp = Fraction(2) ** (e - (p - 1))
    q = abs(x) / ulp
    fl = q.numerator // q.denominator
    rem = q - fl
    if rem > Fraction(1, 2) or (rem == Fraction(1, 2) and fl % 2 == 1):
        fl += 1
    return s * fl * ulp


def _rf32(x):  return _round_frac(x, 24, -126)
def _rbf16(x): return _round_frac(x, 8, -126)


def _bits_t(bits: np.ndarray) -> torch.Tensor:
    return torch.from_numpy(bits.view(np.int16).copy()).view(torch.bfloat16)


def _t_bits(t: torch.Tensor) -> np.ndarray:
    return t.contiguous().view(torch.int16).numpy().view(np.uint16)


# ---------------------------------------------------------------- bf16 conversions
def test_bf16_to_f32_exhaustive_vs_torch():
    bits = np.arange(65536, dtype=np.uint32).astype(np.uint16)
    mine = O.bf16_bits_to_f32(bits)
    ref = _bits_t(bits).float().numpy()
    assert np.array_equal(mine.view(np.uint32), ref.view(np.uint32))


def test_f32_to_bf16_vs_torch_and_ties():
    rng = np.random.default_rng(0)
    u = rng.integers(0, 2**32, size=2_000_000, dtype=np.uint64).astype(np.uint32)
    # add exact ties and near-ties around every bf16 boundary pattern
    hi = rng.integers(0, 2**16, size=100_000, dtype=np.uint64).astype(np.uint32) << np.uint32(16)
    ties = np.concatenate([hi | np.uint32(0x8000), hi | np.uint32(0x7FFF), hi | np.uint32(0x8001)])
    u = np.concatenate([u, ties])
    x = u.view(np.float32)
    finite = np.isfinite(x)
    mine = O.f32_to_bf16_bits(x)
    ref = _t_bits(torch.from_numpy(x.copy()).to(torch.bfloat16))
    assert np.array_equal(mine[finite], ref[finite])
    nan = np.isnan(x)
    assert np.all(np.isnan(O.bf16_bits_to_f32(mine[nan])))


def test_f32_to_bf16_bruteforce_rational():
    rng = np.random.default_rng(1)
    x = (rng.standard_normal(300) * np.float32(3.0)).astype(np.float32)
    got = O.f32_to_bf16_bits(x)
    for xi, g in zip(x, got):
        want = _rbf16(Fraction(float(xi)))
        assert _frac_of_bf16(int(g)) == want


# ---------------------------------------------------------------- reduce
def test_reduce_known_answer_ones():
    """The reference's own check: 8192 bf16 ones on every rank -> 8
    (triton_one_shot_all_reduce.py:145-154)."""
    one = np.full(8192, 0x3F80, dtype=np.uint16)
    out = O.reduce_ref([one] * 8, "bf16")
    assert np.all(O.bf16_bits_to_f32(out) == 8.0)
    out32 = O.reduce_ref([np.ones(8192, np.float32)] * 8, "fp32")
    assert np.all(out32 == 8.0)
    assert np.all(O.bf16_bits_to_f32(O.reduce_ref_bf16_acc([one] * 8)) == 8.0)


def test_reduce_bf16_bruteforce_rational():
    bufs = [O.seeded_normal_bf16_bits(48, seed=r) for r in range(8)]
    got = O.reduce_ref(bufs, "bf16")
    for j in range(48):
        acc = Fraction(0)
        for r in range(8):
            acc = _rf32(acc + _frac_of_bf16(int(bufs[r][j])))
        assert _frac_of_bf16(int(got[j])) == _rbf16(acc), j


def test_reduce_fp32_bruteforce_rational_and_order():
    bufs = [O.seeded_normal_f32(40, seed=r) for r in range(8)]
    got = O.reduce_ref(bufs, "fp32")
    rev = O.reduce_ref(bufs[::-1], "fp32")
    for j in range(40):
        acc = Fraction(0)
        for r in range(8):
            acc = _rf32(acc + Fraction(float(bufs[r][j])))
        assert Fraction(float(got[j])) == acc
    # summation order is observable in fp32: the reverse order differs somewhere
    big = [O.seeded_normal_f32(4096, seed=r) for r in range(8)]
    assert not np.array_equal(O.reduce_ref(big, "fp32"), O.reduce_ref(big[::-1], "fp32"))
    assert rev.shape == got.shape


def test_reduce_vs_torch_cpu():
    n = 1 << 16
    bufs = [O.seeded_normal_bf16_bits(n, seed=r) for r in range(8)]
    acc = torch.zeros(n, dtype=torch.float32)
    for b in bufs:
        acc += _bits_t(b).float()
    assert np.array_equal(O.reduce_ref(bufs, "bf16"), _t_bits(acc.to(torch.bfloat16)))
    f = [O.seeded_normal_f32(n, seed=r) for r in range(8)]
    acc = torch.zeros(n, dtype=torch.float32)
    for b in f:
        acc += torch.from_numpy(b)
    assert np.array_equal(O.reduce_ref(f, "fp32").view(np.uint32), acc.numpy().view(np.uint32))


def test_reduce_invariants():
    n = 4096
    bufs = [O.seeded_normal_bf16_bits(n, seed=r) for r in range(8)]
    base = O.bf16_bits_to_f32(O.reduce_ref(bufs, "bf16"))
    # exact scaling by a power of two (no overflow/underflow at these magnitudes)
    scaled = [O.f32_to_bf16_bits(O.bf16_bits_to_f32(b) * np.float32(16.0)) for b in bufs]
    assert np.array_equal(O.bf16_bits_to_f32(O.reduce_ref(scaled, "bf16")), base * np.float32(16.0))
    # small integers: exact and order independent
    rng = np.random.default_rng(3)
    ints = [O.f32_to_bf16_bits(rng.integers(-16, 17, n).astype(np.float32)) for _ in range(8)]
    exact = sum(O.bf16_bits_to_f32(b).astype(np.int64) for b in ints)
    assert np.array_equal(O.bf16_bits_to_f32(O.reduce_ref(ints, "bf16")).astype(np.int64), exact)
    assert np.array_equal(O.reduce_ref(ints[::-1], "bf16"), O.reduce_ref(ints, "bf16"))


def test_reduce_bf16_acc_chain_bruteforce():
    bufs = [O.seeded_normal_bf16_bits(64, seed=10 + r) for r in range(8)]
    got = O.reduce_ref_bf16_acc(bufs)
    for j in range(64):
        acc = Fraction(0)
        for r in range(8):
            acc = _rbf16(acc + _frac_of_bf16(int(bufs[r][j])))
        assert _frac_of_bf16(int(got[j])) == acc
    # library cross-check: torch CPU bf16 adds round once per step
    t = torch.zeros(64, dtype=torch.bfloat16)
    for b in bufs:
        t = t + _bits_t(b)
    assert np.array_equal(got, _t_bits(t))


def test_bf16_acc_chain_random_bit_patterns_and_nan():
    """Every exponent distance, subnormals and overflow against exact rational
    arithmetic; a NaN anywhere in the chain gives the canonical 0x7FFF."""
    rng = np.random.default_rng(5)
    bufs = [rng.integers(0, 1 << 16, 512).astype(np.uint16) for _ in range(4)]
    got = O.reduce_ref_bf16_acc(bufs)
    big = Fraction(2) ** 128 - Fraction(2) ** 119          # first value that rounds to infinity
    for j in range(512):
        vals = [int(b[j]) for b in bufs]
        fl = [float(O.bf16_bits_to_f32(np.array([v], np.uint16))[0]) for v in vals]
        if any(np.isnan(f) for f in fl):
            assert got[j] == 0x7FFF
            continue
        acc = 0.0
        bad = False
        fr = Fraction(0)
        for f in fl:
            if np.isinf(f) or np.isinf(acc):
                bad = True
                break
            fr = fr + Fraction(f)
            if abs(fr) >= big:
                bad = True
                break
            fr = _rbf16(fr)
            acc = float(fr)
        if bad:
            continue                                       # infinities: covered by the torch cross-check below
        assert _frac_of_bf16(int(got[j])) == fr, j
    t = torch.zeros(512, dtype=torch.bfloat16)
    for b in bufs:
        t = t + _bits_t(b)
    tb = _t_bits(t)
    nan = np.isnan(O.bf16_bits_to_f32(tb))
    assert np.array_equal(np.isnan(O.bf16_bits_to_f32(got)), nan)
    assert np.array_equal(got[~nan], tb[~nan])
    assert np.all(got[nan] == 0x7FFF)


def test_bf16_acc_double_rounding_case():
    """A sum whose fp32 rounding lands on a bf16 tie: single rounding must win."""
    a = np.array([0x3F80], dtype=np.uint16)            # 1.0
    # 2^-8 + 2^-33 as bf16-representable pieces is not one value; use two adds
    b = O.f32_to_bf16_bits(np.array([2.0 ** -8], np.float32))   # exactly half a bf16 ulp of 1.0
    c = O.f32_to_bf16_bits(np.array([2.0 ** -40], np.float32))
    out = O._f64_to_bf16_bits(np.array([1.0 + 2.0 ** -8 + 2.0 ** -40]))
    assert _frac_of_bf16(int(out[0])) == _rbf16(Fraction(1) + Fraction(2) ** -8 + Fraction(2) ** -40)
    assert a.shape == b.shape == c.shape


def test_reduce_grid_formula():
    # triton_one_shot_all_reduce.py:97-109
    assert O.reduce_grid(8192) == 2
    assert O.reduce_grid(8) == 1
    assert O.reduce_grid(512 * 8 * 24) == 24
    assert O.reduce_grid(1 << 25) == 24


# ---------------------------------------------------------------- barrier
def test_barrier_slots():
    send, wait = O.barrier_slots(block_id=5, rank=3, world_size=8)
    assert send == [(r, 43) for r in range(8)]
    assert wait == [(3, 40 + r) for r in range(8)]
    # every slot of block b is written by exactly one (sender, receiver) pair
    seen = set()
    for rank in range(8):
        s, _ = O.barrier_slots(7, rank, 8)
        for slot in s:
            assert slot not in seen
            seen.add(slot)
    assert len(seen) == 64


@pytest.mark.parametrize("ws,rounds", [(2, 3), (3, 2)])
def test_barrier_model_exhaustive(ws, rounds):
    terminals, nstates = O.BarrierModel(ws, rounds).explore()
    assert nstates > 10
    assert len(terminals) == 1
    pads, pcs = next(iter(terminals))
    assert all(v == 0 for v in pads), "pads must be all-zero after the barrier (triton_barrier.py:60-65)"


def test_barrier_model_detects_stale_pad():
    m = O.BarrierModel(2, 1)
    pads, pcs = m.initial()
    pads = list(pads); pads[1] = 1            # stale flag rank 1 -> rank 0 left behind
    with pytest.raises(AssertionError):
        # rank 0 may consume the stale flag before rank 1 sends: barrier property broken
        seen = {(tuple(pads), pcs)}
        stack = [(tuple(pads), pcs)]
        while stack:
            s = stack.pop()
            nxt = m.steps(s)
            if not nxt and not all(pc == 2 for pc in s[1]):
                raise AssertionError("deadlock")
            for t in nxt:
                if t not in seen:
                    seen.add(t); stack.append(t)


# ---------------------------------------------------------------- all-gather
def test_all_gather_order_and_result():
    assert O.all_gather_order(3, 8) == [4, 5, 6, 7, 0, 1, 2, 3]
    assert O.all_gather_order(0, 8) == [1, 2, 3, 4, 5, 6, 7, 0]
    assert O.all_gather_order(1, 4, 2) == [4, 5, 6, 7, 0, 1, 2, 3]
    shards = [np.full((4, 6), r, dtype=np.uint16) for r in range(8)]
    out, prog, order = O.all_gather_ref(shards, rank=2)
    assert out.shape == (32, 6)
    for r in range(8):
        assert np.all(out[4 * r:4 * r + 4] == r)
    assert np.all(prog == 1) and sorted(order) == list(range(8))


# ---------------------------------------------------------------- tile schedule
def _flatten(sched):
    return [t for p in sorted(sched) for t in sched[p]]


@pytest.mark.parametrize("rank", [0, 3, 7])
def test_ref_schedule_properties_config5(rank):
    M, N, BM, BN, G = 16384, 3584, 256, 128, 4
    sched = O.ref_tile_schedule(M, N, BM, BN, G, comm_block_m=2048, rank=rank, world_size=8,
                                num_programs=256)
    tiles = _flatten(sched)
    assert len(tiles) == 1792
    assert len({(t["pid_m"], t["pid_n"]) for t in tiles}) == 1792       # bijection
    for p, lst in sched.items():
        assert len(lst) == 7
        # the first 256 tiles span 2.3 swizzle groups = rows 0..2559 past the pivot:
        # the local shard and the first quarter of the next one
        assert (lst[0]["comm_block"] - rank) % 8 in (0, 1)
        # comm blocks are first touched in ring order starting at the local rank
        ring = [(t["comm_block"] - rank) % 8 for t in lst]
        assert ring == sorted(ring)
    for t in tiles:
        assert t["local"] == (t["comm_block"] == rank)                   # local tiles never wait
        if t["local"]:
            assert 0 <= t["a_row"] < 2048 and t["a_row"] == t["pid_m"] * BM - rank * 2048
        else:
            assert t["a_row"] == t["pid_m"] * BM
    if rank == 3:
        waves = [sorted({sched[p][i]["comm_block"] for p in sched}) for i in range(7)]
        assert waves == [[3, 4], [4, 5], [5, 6], [6, 7], [0, 7], [0, 1], [1, 2]]


def test_ref_schedule_small_shapes_bijection():
    for (M, N, BM, BN, G, ws, progs) in [(512, 256, 64, 64, 2, 4, 7), (1024, 384, 128, 128, 1, 8, 5),
                                         (2048, 512, 128, 64, 2, 8, 304)]:
        comm = M // ws
        assert comm % (BM * G) == 0       # triton_all_gather_matmul.py:244
        for rank in range(ws):
            tiles = _flatten(O.ref_tile_schedule(M, N, BM, BN, G, comm, rank, ws, progs))
            assert len({(t["pid_m"], t["pid_n"]) for t in tiles}) == (M // BM) * (N // BN) == len(tiles)


# ---------------------------------------------------------------- matmul / gemv
def test_ag_matmul_vs_torch_and_bruteforce():
    shards = [O.seeded_normal_bf16_bits(8 * 32, seed=r, std=0.02).reshape(8, 32) for r in range(4)]
    b = O.seeded_normal_bf16_bits(16 * 32, seed=100, std=0.02).reshape(16, 32)
    bits, c32 = O.ag_matmul_ref(shards, b, return_f32=True)
    a_t = torch.cat([_bits_t(s) for s in shards]).float()
    ref = (a_t @ _bits_t(b).float().T)
    # fp32 dot products of 32 terms: library and numpy may associate differently
    assert np.allclose(c32, ref.numpy(), rtol=1e-5, atol=1e-9)
    # exact rational: the bf16 result may differ from the exactly-rounded one only
    # when the fp32 sum sits within fp32 rounding error of a bf16 tie
    A = np.concatenate(shards)
    nbad = 0
    for i in range(0, 32, 5):
        for j in range(16):
            exact = sum(_frac_of_bf16(int(A[i, k])) * _frac_of_bf16(int(b[j, k])) for k in range(32))
            if _frac_of_bf16(int(bits[i, j])) != _rbf16(exact):
                nbad += 1
                assert abs(Fraction(float(c32[i, j])) - exact) <= abs(exact) * Fraction(1, 1 << 18) + Fraction(2) ** -40
    assert nbad <= 2


def test_gemv_ref_vs_library_and_bruteforce():
    x = O.seeded_normal_bf16_bits(2 * 64, seed=0).reshape(2, 64)
    w = O.seeded_normal_bf16_bits(64 * 24, seed=1, std=0.02).reshape(64, 24)
    out, partials = O.gemv_allreduce_ref(x, w, world_size=8, return_partials=True)
    assert partials.shape == (8, 2, 24)
    ref = _bits_t(x).float() @ _bits_t(w).float()
    got = O.bf16_bits_to_f32(out)
    assert np.allclose(got, ref.numpy(), rtol=2 ** -7, atol=1e-6)   # within 1 bf16 ulp of x @ W
    for r in range(8):                                             # partials exact to fp32 rounding
        for j in range(0, 24, 7):
            exact = sum(_frac_of_bf16(int(x[1, r * 8 + k])) * _frac_of_bf16(int(w[r * 8 + k, j]))
                        for k in range(8))
            assert Fraction(float(partials[r, 1, j])) == _rf32(exact)
    for j in range(24):                                            # rank-ordered fp32 combine
        acc = Fraction(0)
        for r in range(8):
            acc = _rf32(acc + Fraction(float(partials[r, 0, j])))
        assert _frac_of_bf16(int(out[0, j])) == _rbf16(acc)


# ---------------------------------------------------------------- signal round
def test_signal_round_ref_bruteforce():
    rng = np.random.default_rng(5)
    src = rng.integers(0, 2**32, size=(3, 4, 16), dtype=np.uint64).astype(np.uint32)
    for rnd in (0, 1, 9999, 2**31):
        want = np.zeros(4, dtype=np.uint32)
        for b in range(4):
            s = 0
            for r in range(3):
                for w in src[r, b]:
                    s = (s + ((int(w) + rnd) & 0xFFFFFFFF)) & 0xFFFFFFFF
            want[b] = s
        assert np.array_equal(O.signal_round_ref(src, rnd), want)


# ---------------------------------------------------------------- fp8 (e4m3fn)
def test_fp8_decode_exhaustive_vs_torch():
    bits = np.arange(256, dtype=np.uint8)
    mine = O.fp8_e4m3fn_to_f32(bits)
    ref = torch.from_numpy(bits.copy()).view(torch.float8_e4m3fn).float().numpy()
    nan = np.isnan(ref)
    assert np.array_equal(np.isnan(mine), nan) and set(bits[nan]) == {0x7F, 0xFF}
    assert np.array_equal(mine[~nan].view(np.uint32), ref[~nan].view(np.uint32))


def test_fp8_encode_vs_torch_ties_and_saturation():
    pos = O.fp8_e4m3fn_to_f32(np.arange(127, dtype=np.uint8)).astype(np.float64)
    mids = (pos[:-1] + pos[1:]) / 2
    rng = np.random.default_rng(9)
    x = np.concatenate([pos, mids, np.nextafter(mids.astype(np.float32), 0), np.nextafter(mids.astype(np.float32), 1e9),
                        rng.standard_normal(200000) * 3, rng.uniform(-448, 448, 200000),
                        rng.uniform(-2 ** -6, 2 ** -6, 100000)]).astype(np.float32)
    x = np.concatenate([x, -x])
    mine = O.f32_to_fp8_e4m3fn(x)
    ref = torch.from_numpy(x).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    assert np.array_equal(mine, ref)                                    # |x| <= 448: one answer
    # exact values round-trip; ties go to the even code
    assert np.array_equal(O.f32_to_fp8_e4m3fn(pos.astype(np.float32)), np.arange(127, dtype=np.uint8))
    assert np.all(O.f32_to_fp8_e4m3fn(mids.astype(np.float32)) % 2 == 0)
    # beyond the largest finite value: saturate (cvt.rn.satfinite), NaN stays NaN
    big = np.array([449, 464, 465, 480, 1e6, np.inf, -500, -np.inf, np.nan], dtype=np.float32)
    assert O.f32_to_fp8_e4m3fn(big).tolist() == [126, 126, 126, 126, 126, 126, 254, 254, 0x7F]


def test_fp8_matmul_vs_torch_cpu():
    rng = np.random.default_rng(2)
    a = rng.integers(0, 256, (48, 128)).astype(np.uint8)
    b = rng.integers(0, 256, (40, 128)).astype(np.uint8)
    a[(a & 0x7F) == 0x7F] = 0x38                                         # no NaN operands
    b[(b & 0x7F) == 0x7F] = 0x38
    a = np.where((a & 0x78) > 0x50, a & 0xCF, a)                         # keep sums finite and below 448 often
    got, c = O.ag_matmul_ref_fp8([a[:24], a[24:]], b, return_f32=True)
    ta = torch.from_numpy(a.copy()).view(torch.float8_e4m3fn).float()
    tb = torch.from_numpy(b.copy()).view(torch.float8_e4m3fn).float()
    tc = ta @ tb.T
    assert np.allclose(c, tc.numpy(), rtol=1e-6, atol=1e-6)
    inr = np.abs(c) <= 448
    want = tc.to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    # identical except where the two fp32 sums straddle a rounding boundary
    same = got[inr] == want[inr]
    assert same.mean() > 0.999
    assert np.all(got[~inr] & 0x7F == 126)


def test_torch_restatement_of_the_reduce_matches_the_numpy_oracle():
    """oracle/torch_reduce.py (what the benchmark times on the CPU) against reduce_ref, bit for
    bit: N(0,1) data, random bit patterns with infinities and denormals, and fp32 buffers."""
    import torch
    from oracle import torch_reduce as T
    rng = np.random.default_rng(7)
    n = 4096
    bits = [O.seeded_normal_bf16_bits(n, seed=r) for r in range(8)]
    tens = [torch.from_numpy(b.view(np.int16).copy()).view(torch.bfloat16) for b in bits]
    got = T.reduce_ref_torch(tens).view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(got, O.reduce_ref(bits, "bf16"))
    raw = [rng.integers(0, 1 << 16, size=n, dtype=np.uint16) for _ in range(8)]
    tens = [torch.from_numpy(b.view(np.int16).copy()).view(torch.bfloat16) for b in raw]
    got = T.reduce_ref_torch(tens).view(torch.int16).numpy().view(np.uint16)
    want = O.reduce_ref(raw, "bf16")
    nan = np.isnan(O.bf16_bits_to_f32(want))
    assert np.array_equal(np.isnan(O.bf16_bits_to_f32(got)), nan) and np.array_equal(got[~nan], want[~nan])
    f = [rng.standard_normal(n).astype(np.float32) for _ in range(8)]
    got = T.reduce_ref_torch([torch.from_numpy(x.copy()) for x in f]).numpy()
    assert np.array_equal(got.view(np.uint32), O.reduce_ref(f, "fp32").view(np.uint32))
    # the per-rank generator of the benchmark's CPU leg is deterministic
    assert torch.equal(T.seeded_normal(64, 3), T.seeded_normal(64, 3))
