"""CPU oracle for the symmetric-memory hot path.  TEST INFRASTRUCTURE ONLY.

This module is the checker the GPU kernels are compared against.  It is imported
only by tests, by the smoke check and by the benchmark's CPU-baseline leg; the
shipped package never imports it and has no CPU fallback.

Everything is restated from the reference's algorithm with numpy integer/float
arithmetic (no torch on the arithmetic path, so that torch-CPU can serve as an
independent cross-check in the tests):

* ``bf16_bits_to_f32`` / ``f32_to_bf16_bits``   bf16 <-> fp32 conversion (RNE)
* ``reduce_ref``           one-shot all-reduce arithmetic
                           (symm_mem_recipes/triton_one_shot_all_reduce.py:77-93:
                           accumulator starts at +0, peers added in rank order
                           0..world_size-1).  Accumulation is fp32 with one
                           final rounding (the build's stated deviation from
                           the reference's per-step bf16 rounding, :36-49).
* ``reduce_ref_bf16_acc``  the reference's own per-step bf16-rounded chain
                           (triton_one_shot_all_reduce.py:32-56), as a
                           correctly-rounded add of two bf16 per step.
* ``reduce_grid``          host grid formula (triton_one_shot_all_reduce.py:97-109)
* ``barrier_slots``        signal-pad slot indexing (triton_barrier.py:100-110)
* ``BarrierModel``         interleaving model of the CAS handshake
                           (triton_barrier.py:112-139)
* ``all_gather_ref``       producer copy order + progress flags
                           (triton_all_gather_matmul.py:41-55)
* ``ref_tile_schedule``    persistent tile walk, grouped swizzle, rank pivot,
                           local/remote source select
                           (triton_all_gather_matmul.py:125-174)
* ``ag_matmul_ref``        cat + matmul (triton_all_gather_matmul.py:322-326),
                           NT layout and fp32 accumulate / bf16 store (:176-193)
* ``ag_matmul_ref_fp8``    the same product with e4m3fn operands and result (the
                           reference's FP8_OUTPUT switch, :115,123,188), with
                           ``fp8_e4m3fn_to_f32`` / ``f32_to_fp8_e4m3fn``
* ``gemv_allreduce_ref``   split-K GEMV + rank-ordered fp32 combine (no
                           reference code exists for it; closed form)
* ``signal_round_ref``     checksum closed form for the producer/consumer
                           signal-pad round benchmark

Pinning status (what the tests check each function against, other than itself):
  bf16 conversions   -> torch CPU casts (library), exhaustive over all 65536 bf16
                        patterns one way, brute-force integer rounding the other
  reduce_ref         -> the reference's known answer ones -> world_size at
                        numel 8192 (triton_one_shot_all_reduce.py:145-154),
                        exact-rational brute force (fractions.Fraction) on small
                        inputs, torch-CPU sequential fp32 adds, scaling by 2^k,
                        small-integer order independence
  reduce_ref_bf16_acc-> exact-rational brute force per step, torch-CPU bf16 adds
  BarrierModel       -> exhaustive interleavings (world_size 2 and 3, two
                        rounds): termination, all-zero pads, barrier property
  all_gather_ref     -> closed form a_out == cat(shards); flag order rank+1..rank
  ref_tile_schedule  -> bijection / ring-order / local-never-waits properties and
                        the per-wave comm-block sets stated for the 16384x3584
                        shape with 256x128 tiles
  ag_matmul_ref      -> torch-CPU matmul (library), exact-rational brute force on
                        tiny shapes; the reference's own check is allclose against
                        all-gather + matmul (triton_all_gather_matmul.py:390-392)
  fp8 conversions    -> torch CPU casts (library): decode exhaustive over all 256
                        patterns, encode on random values, every midpoint and
                        every representable value up to 448; beyond 448 torch
                        gives NaN where the reference's hardware conversion
                        saturates (PTX cvt.rn.satfinite): that branch is PARITY
                        UNPINNED against the reference's toolchain and follows
                        the published PTX semantics
  ag_matmul_ref_fp8  -> torch-CPU matmul of the decoded operands + torch cast
  gemv_allreduce_ref -> PARITY UNPINNED against the reference (no reference code
                        or vectors exist for this path); pinned only against
                        the mathematics: x @ W library routine and
                        exact-rational brute force on tiny shapes
  signal_round_ref   -> brute force on a tiny slab
"""
from __future__ import annotations

import itertools
from typing import Dict, List, Sequence, Tuple

import numpy as np

WORLD_SIZE = 8


# --------------------------------------------------------------------------
# bf16 <-> fp32 on raw bit patterns
# --------------------------------------------------------------------------
def bf16_bits_to_f32(bits: np.ndarray) -> np.ndarray:
    """uint16 bf16 patterns -> float32 (exact: bf16 is the top half of fp32)."""
    bits = np.ascontiguousarray(bits, dtype=np.uint16)
    return (bits.astype(np.uint32) << np.uint32(16)).view(np.float32)


def f32_to_bf16_bits(x: np.ndarray) -> np.ndarray:
    """float32 -> uint16 bf16 patterns, round-to-nearest-even; NaN stays NaN."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    u = x.view(np.uint32)
    lsb = (u >> np.uint32(16)) & np.uint32(1)
    rounded = (u + np.uint32(0x7FFF) + lsb) >> np.uint32(16)
    is_nan = (u & np.uint32(0x7FFFFFFF)) > np.uint32(0x7F800000)
    quiet = (u >> np.uint32(16)) | np.uint32(0x0040)
    return np.where(is_nan, quiet, rounded).astype(np.uint16)


# --------------------------------------------------------------------------
# one-shot all-reduce
# --------------------------------------------------------------------------
def reduce_ref(bufs: Sequence[np.ndarray], dtype: str) -> np.ndarray:
    """Sum ``world_size`` peer buffers element-wise in rank order.

    ``dtype`` is "bf16" (buffers are uint16 bit patterns, result uint16 bit
    patterns) or "fp32" (float32 in, float32 out).  The accumulator is fp32 +0
    and the peers are added one at a time, rank 0 first
    (triton_one_shot_all_reduce.py:84-89).  For bf16 the sum is rounded to
    bf16 once, at the end.
    """
    assert dtype in ("bf16", "fp32")
    n = bufs[0].shape[0]
    acc = np.zeros(n, dtype=np.float32)
    for b in bufs:
        assert b.shape == (n,)
        v = bf16_bits_to_f32(b) if dtype == "bf16" else np.asarray(b, dtype=np.float32)
        acc = (acc + v).astype(np.float32)
    return f32_to_bf16_bits(acc) if dtype == "bf16" else acc


def reduce_ref_bf16_acc(bufs: Sequence[np.ndarray]) -> np.ndarray:
    """The reference's accumulate-in-bf16 chain (triton_one_shot_all_reduce.py:36-49).

    Each step is one correctly rounded bf16 add.  The fp32 sum of two bf16
    values is exact whenever their exponents differ by < 16, and otherwise the
    fp32 rounding cannot move the result across a bf16 rounding boundary except
    in double-rounding ties; those are resolved by doing the add in float64
    (53-bit significand holds any sum of two bf16 exactly unless exponents
    differ by > 44, where the small operand is below half an ulp of bf16 and a
    sticky bit suffices) and rounding once to bf16.
    """
    n = bufs[0].shape[0]
    acc = np.zeros(n, dtype=np.uint16)
    for b in bufs:
        with np.errstate(invalid="ignore"):
            s = bf16_bits_to_f32(acc).astype(np.float64) + bf16_bits_to_f32(b).astype(np.float64)
        acc = _f64_to_bf16_bits(s)
        # add.bf16x2 returns the canonical NaN 0x7FFF whatever the operands' payloads
        # (PTX ISA 8.x, "Half Precision Floating-Point Instructions: add"; the CUDA
        # toolkit is a third-party dependency that is not part of the reference tree)
        acc = np.where(np.isnan(s), np.uint16(0x7FFF), acc).astype(np.uint16)
    return acc


def _f64_to_bf16_bits(x: np.ndarray) -> np.ndarray:
    """float64 -> bf16 bits with a single RNE rounding (no fp32 intermediate)."""
    x = np.ascontiguousarray(x, dtype=np.float64)
    # Round-to-odd into fp32, then RNE to bf16: round-to-odd keeps a sticky bit
    # so the second rounding behaves like a single one (fp32 has > 2 extra bits).
    f = x.astype(np.float32)
    back = f.astype(np.float64)
    inexact = back != x
    u = f.view(np.uint32).copy()
    # move toward zero when the cast rounded away from zero, then force lsb odd
    away = inexact & (np.abs(back) > np.abs(x))
    u = np.where(away, u - np.uint32(1), u)
    u = np.where(inexact, u | np.uint32(1), u)
    finite = np.isfinite(x)
    u = np.where(finite, u, f.view(np.uint32))
    return f32_to_bf16_bits(u.astype(np.uint32).view(np.float32))


def reduce_grid(numel: int, numel_per_thread: int = 8, block_size: int = 512,
                max_blocks: int = 24) -> int:
    """Reference grid size (triton_one_shot_all_reduce.py:97-109)."""
    cdiv = lambda a, b: -(-a // b)
    return min(cdiv(cdiv(numel, numel_per_thread), block_size), max_blocks)


# --------------------------------------------------------------------------
# blockwise barrier
# --------------------------------------------------------------------------
def barrier_slots(block_id: int, rank: int, world_size: int) -> Tuple[List[Tuple[int, int]], List[Tuple[int, int]]]:
    """(pad, index) pairs a rank's block touches (triton_barrier.py:100-110).

    send[r] = slot ``block_id*world_size + rank`` on peer r's pad,
    wait[r] = slot ``block_id*world_size + r`` on the rank's own pad.
    """
    send = [(r, block_id * world_size + rank) for r in range(world_size)]
    wait = [(rank, block_id * world_size + r) for r in range(world_size)]
    return send, wait


class BarrierModel:
    """Sequentially consistent interleaving model of the CAS handshake.

    One "thread" per (rank, lane) pair, as in triton_barrier.py:112-139: lane r
    of rank k first spins on CAS(pad[r][slot(k)], 0 -> 1), then spins on
    CAS(pad[k][slot(r)], 1 -> 0).  A rank leaves the barrier when all of its
    lanes have finished (the bar.sync at :141-143).  ``rounds`` back-to-back
    barriers are run with no reset of the pads in between.

    ``explore`` walks every reachable state (spinning steps that do not change
    the state are dropped, so the walk is finite) and returns the set of
    terminal states; it raises if a non-terminal state has no enabled step
    (deadlock) or if the barrier property is violated: a rank may only finish
    round n after every rank has entered round n.
    """

    def __init__(self, world_size: int, rounds: int = 2):
        self.ws = world_size
        self.rounds = rounds

    def initial(self):
        ws = self.ws
        pads = tuple(0 for _ in range(ws * ws))  # pads[k*ws + r]: slot r of rank k's pad
        # per (rank, lane): program counter = 2*round + phase (0 = send, 1 = wait)
        pcs = tuple(0 for _ in range(ws * ws))
        return pads, pcs

    def _rank_round(self, pcs, k):
        """Round rank k is currently in = min over its lanes (bar.sync)."""
        ws = self.ws
        return min(pcs[k * ws + r] // 2 for r in range(ws))

    def steps(self, state):
        pads, pcs = state
        ws = self.ws
        out = []
        for k in range(ws):
            rank_round = self._rank_round(pcs, k)
            for r in range(ws):
                pc = pcs[k * ws + r]
                rnd, phase = divmod(pc, 2)
                if rnd >= self.rounds:
                    continue
                if rnd > rank_round:
                    continue  # lane waits at the block barrier for its siblings
                if phase == 0:
                    idx = r * ws + k  # peer r's pad, slot for sender k
                    if pads[idx] == 0:
                        np_ = list(pads); np_[idx] = 1
                        npc = list(pcs); npc[k * ws + r] = pc + 1
                        out.append((tuple(np_), tuple(npc)))
                else:
                    idx = k * ws + r  # own pad, slot for sender r
                    if pads[idx] == 1:
                        # barrier property: sender r must have entered this round
                        assert pcs[r * ws + k] > 2 * rnd, "flag seen before peer sent it"
                        np_ = list(pads); np_[idx] = 0
                        npc = list(pcs); npc[k * ws + r] = pc + 1
                        out.append((tuple(np_), tuple(npc)))
        return out

    def explore(self):
        start = self.initial()
        seen = {start}
        stack = [start]
        terminals = set()
        done_pc = 2 * self.rounds
        while stack:
            s = stack.pop()
            nxt = self.steps(s)
            if not nxt:
                if all(pc == done_pc for pc in s[1]):
                    terminals.add(s)
                    continue
                raise AssertionError(f"deadlock in state {s}")
            for t in nxt:
                if t not in seen:
                    seen.add(t)
                    stack.append(t)
        return terminals, len(seen)


# --------------------------------------------------------------------------
# all-gather producer
# --------------------------------------------------------------------------
def all_gather_order(rank: int, world_size: int, splits_per_rank: int = 1) -> List[int]:
    """Progress-flag indices in the order the producer sets them
    (triton_all_gather_matmul.py:43-55): sources rank+1, ..., rank+world_size-1,
    rank; within a source, splits in increasing order."""
    order = []
    for step in range(world_size):
        src = (rank + step + 1) % world_size
        for split in range(splits_per_rank):
            order.append(src * splits_per_rank + split)
    return order


def all_gather_ref(shards: Sequence[np.ndarray], rank: int, splits_per_rank: int = 1):
    """Returns (gathered, progress, order).  ``gathered`` is the row-wise
    concatenation of the shards (chunk src*splits+s of the output receives chunk s
    of peer src's shard, triton_all_gather_matmul.py:41-49) and every progress
    flag ends at 1."""
    ws = len(shards)
    out = np.concatenate([np.asarray(s) for s in shards], axis=0)
    progress = np.ones(ws * splits_per_rank, dtype=np.uint32)
    return out, progress, all_gather_order(rank, ws, splits_per_rank)


# --------------------------------------------------------------------------
# tile schedule of the reference's persistent GEMM
# --------------------------------------------------------------------------
def ref_tile_schedule(M: int, N: int, BM: int, BN: int, group_m: int, comm_block_m: int,
                      rank: int, world_size: int, num_programs: int) -> Dict[int, List[dict]]:
    """Per-program list of tiles in visiting order
    (triton_all_gather_matmul.py:125-174).

    Each entry: pid_m, pid_n (output tile, after the pivot), comm_block, local
    (True: rows come from the local shard, no wait), a_row (row offset inside
    the source: shard-relative when local, gathered-buffer row otherwise).
    """
    cdiv = lambda a, b: -(-a // b)
    num_pid_m = cdiv(M, BM)
    num_pid_n = cdiv(N, BN)
    num_tiles = num_pid_m * num_pid_n
    num_pid_in_group = group_m * num_pid_n
    n_comm = M // comm_block_m
    n_comm_per_rank = n_comm // world_size
    pid_m_per_comm = comm_block_m // BM
    sched: Dict[int, List[dict]] = {}
    for p in range(min(num_programs, num_tiles)):
        tiles = []
        tile_id = p
        while tile_id < num_tiles:
            group_id = tile_id // num_pid_in_group
            first_pid_m = group_id * group_m
            gsm = min(num_pid_m - first_pid_m, group_m)
            pid_m = first_pid_m + (tile_id % gsm)
            pid_n = (tile_id % num_pid_in_group) // gsm
            pid_m = (pid_m + pid_m_per_comm * rank) % num_pid_m
            comm_block = pid_m // pid_m_per_comm
            local = (comm_block // n_comm_per_rank) == rank
            a_row = (pid_m * BM) % comm_block_m if local else pid_m * BM
            tiles.append(dict(pid_m=pid_m, pid_n=pid_n, comm_block=comm_block,
                              local=local, a_row=a_row))
            tile_id += num_programs
        sched[p] = tiles
    return sched


# --------------------------------------------------------------------------
# all-gather matmul arithmetic
# --------------------------------------------------------------------------
def ag_matmul_ref(shards_bits: Sequence[np.ndarray], b_nk_bits: np.ndarray,
                  return_f32: bool = False):
    """C[M,N] = cat(shards)[M,K] @ B[N,K]^T, fp32 accumulate, bf16 result
    (triton_all_gather_matmul.py:322-326 and :176-193).  Inputs are uint16 bf16
    bit patterns; returns uint16 bf16 bit patterns (and the fp32 product when
    ``return_f32``)."""
    a = bf16_bits_to_f32(np.concatenate(list(shards_bits), axis=0))
    b = bf16_bits_to_f32(b_nk_bits)
    c = a @ b.T
    bits = f32_to_bf16_bits(c)
    return (bits, c) if return_f32 else bits


# --------------------------------------------------------------------------
# fp8 (e4m3fn) variant of the matmul: FP8_OUTPUT, triton_all_gather_matmul.py:115,123,188
# --------------------------------------------------------------------------
def fp8_e4m3fn_to_f32(bits: np.ndarray) -> np.ndarray:
    """uint8 e4m3fn patterns -> float32 (OCP FP8: bias 7, no infinities, S.1111.111 = NaN)."""
    b = np.ascontiguousarray(bits, dtype=np.uint8).astype(np.int32)
    sign = np.where(b & 0x80, -1.0, 1.0)
    e = (b >> 3) & 0xF
    m = b & 0x7
    val = np.where(e == 0, m * 2.0 ** -9, (8 + m) * 2.0 ** (e - 10.0))
    val = np.where((e == 15) & (m == 7), np.nan, val)
    return (sign * val).astype(np.float32)


_FP8_POS = None


def f32_to_fp8_e4m3fn(x: np.ndarray) -> np.ndarray:
    """float32 -> uint8 e4m3fn, round to nearest even, saturating to +-448 (also for
    infinities), NaN -> 0x7F: what Triton's cast to float8e4nv compiles to on the
    reference's hardware, ``cvt.rn.satfinite.e4m3x2.f32`` (PTX ISA 8.x, "cvt"; the
    CUDA toolkit is a third-party dependency outside the reference tree)."""
    global _FP8_POS
    if _FP8_POS is None:
        _FP8_POS = fp8_e4m3fn_to_f32(np.arange(127, dtype=np.uint8)).astype(np.float64)   # 0 .. 448
    x = np.ascontiguousarray(x, dtype=np.float32)
    a = np.abs(x).astype(np.float64)
    hi = np.clip(np.searchsorted(_FP8_POS, a, side="left"), 1, 126)       # first code with value >= a
    lo = hi - 1
    dlo = a - _FP8_POS[lo]
    dhi = _FP8_POS[hi] - a
    code = np.where(dlo < dhi, lo, np.where(dhi < dlo, hi, np.where(lo % 2 == 0, lo, hi)))
    code = np.where(a >= 448.0, 126, code)                                 # satfinite, infinities too
    code = np.where(a == 0.0, 0, code)
    out = (code | np.where(np.signbit(x), 0x80, 0)).astype(np.uint8)
    return np.where(np.isnan(x), np.uint8(0x7F), out).astype(np.uint8)


def ag_matmul_ref_fp8(shards_bits: Sequence[np.ndarray], b_nk_bits: np.ndarray, return_f32: bool = False):
    """C = cat(shards) @ B^T with e4m3fn operands, fp32 accumulate, e4m3fn result
    (triton_all_gather_matmul.py:123 dtype switch, :176-188).  uint8 in, uint8 out."""
    a = fp8_e4m3fn_to_f32(np.concatenate(list(shards_bits), axis=0))
    b = fp8_e4m3fn_to_f32(b_nk_bits)
    c = a @ b.T
    bits = f32_to_fp8_e4m3fn(c)
    return (bits, c) if return_f32 else bits


def seeded_normal_fp8_bits(n: int, seed: int, std: float = 1.0) -> np.ndarray:
    """N(0, std) from numpy's PCG64 seeded per tensor, rounded to e4m3fn."""
    rng = np.random.default_rng(seed)
    return f32_to_fp8_e4m3fn((rng.standard_normal(n) * std).astype(np.float32))


# --------------------------------------------------------------------------
# split-K GEMV + all-reduce
# --------------------------------------------------------------------------
def gemv_allreduce_ref(x_bits: np.ndarray, w_bits: np.ndarray, world_size: int = WORLD_SIZE,
                       return_partials: bool = False):
    """x [batch,K] bf16, W [K,N] bf16 split into ``world_size`` K-shards.

    partial_r = x[:, shard r] @ W[shard r, :] in fp32 (float64 accumulation
    here, rounded to fp32, so that the oracle does not depend on a summation
    order inside the shard); out = bf16(((0 + p_0) + p_1) + ... + p_{ws-1}).
    """
    x = bf16_bits_to_f32(x_bits).astype(np.float64)
    w = bf16_bits_to_f32(w_bits).astype(np.float64)
    K = x.shape[1]
    ks = K // world_size
    partials = np.stack([(x[:, r * ks:(r + 1) * ks] @ w[r * ks:(r + 1) * ks, :]).astype(np.float32)
                         for r in range(world_size)])
    acc = np.zeros(partials.shape[1:], dtype=np.float32)
    for r in range(world_size):
        acc = (acc + partials[r]).astype(np.float32)
    out = f32_to_bf16_bits(acc)
    return (out, partials) if return_partials else out


# --------------------------------------------------------------------------
# producer/consumer signal round
# --------------------------------------------------------------------------
def signal_round_ref(src_words: np.ndarray, round_idx: int) -> np.ndarray:
    """Checksums of one producer/consumer round.

    ``src_words``: uint32 [world_size, num_blocks, words_per_chunk] (the bf16
    payload viewed as 32-bit words).  In round ``round_idx`` producer (r, b)
    publishes ``src_words[r, b] + round_idx`` (wrapping add per word); consumer
    block b of every rank sums all words of the world_size chunks of block b
    (wrapping uint32).  Returns uint32 [num_blocks].
    """
    ws, nb, wpc = src_words.shape
    base = src_words.astype(np.uint64).sum(axis=(0, 2))
    total = base + np.uint64(ws * wpc) * np.uint64(round_idx)
    return (total & np.uint64(0xFFFFFFFF)).astype(np.uint32)


# --------------------------------------------------------------------------
# seeded inputs shared by tests, smoke and bench (torch generator, CPU)
# --------------------------------------------------------------------------
def seeded_normal_bf16_bits(n: int, seed: int, std: float = 1.0) -> np.ndarray:
    """N(0, std) generated in fp32 on the CPU with torch's generator seeded with
    ``seed`` and rounded to bf16; returned as uint16 bit patterns."""
    import torch
    g = torch.Generator().manual_seed(seed)
    t = (torch.randn(n, generator=g, dtype=torch.float32) * std).to(torch.bfloat16)
    return t.view(torch.int16).numpy().view(np.uint16).copy()


def seeded_normal_f32(n: int, seed: int, std: float = 1.0) -> np.ndarray:
    import torch
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(n, generator=g, dtype=torch.float32) * std).numpy().copy()
