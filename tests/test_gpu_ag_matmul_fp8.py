"""GPU parity of the e4m3fn all-gather matmul (the reference's FP8_OUTPUT switch,
symm_mem_recipes/triton_all_gather_matmul.py:115,123,188,311) against the CPU oracle.

Bar: the fp32 sums differ from the oracle's only by the order of addition, so after
the cast to e4m3fn (3 mantissa bits) almost every entry is bit-identical; an entry
whose sum lies next to a rounding boundary may land on the neighbouring code.  The
test demands >= 99.8 % identical codes and no entry further than one code away."""
import numpy as np
import pytest
import torch

from oracle import oracle as O

pytestmark = pytest.mark.gpu


def _t(bits):
    return torch.from_numpy(bits.copy()).view(torch.float8_e4m3fn)


def _bits(t):
    return t.contiguous().view(torch.uint8).cpu().numpy()


def _setup(M, N, K, ws, rank, cuda, std=0.25):
    from symm_mem_recipes import EmulatedSymmetricMemory as SM
    a_shard = SM.empty_strided_p2p((M // ws, K), (K, 1), torch.float8_e4m3fn, cuda, world_size=ws, rank=rank)
    h = SM.rendezvous(a_shard)
    shards = []
    for r in range(ws):
        bits = O.seeded_normal_fp8_bits(M // ws * K, seed=r, std=std).reshape(M // ws, K)
        h.get_buffer(r, (M // ws, K), torch.uint8).copy_(torch.from_numpy(bits))
        shards.append(bits)
    b_bits = O.seeded_normal_fp8_bits(N * K, seed=100, std=std).reshape(N, K)
    b = _t(b_bits).to(cuda)
    a_out = torch.zeros((M, K), dtype=torch.uint8, device=cuda).view(torch.float8_e4m3fn)
    c_out = torch.full((M, N), 0x7F, dtype=torch.uint8, device=cuda).view(torch.float8_e4m3fn)
    return a_shard, h, shards, b, b_bits, a_out, c_out


def _check(got, want):
    """Codes compared as sign-magnitude integers: neighbouring values differ by 1."""
    assert not np.any((got & 0x7F) == 0x7F), "NaN in the result"
    key = lambda x: np.where(x & 0x80, -(x & 0x7F).astype(np.int32), (x & 0x7F).astype(np.int32))
    d = np.abs(key(got) - key(want))
    assert d.max() <= 1, int(d.max())
    assert np.mean(d == 0) >= 0.998, float(np.mean(d == 0))


@pytest.fixture(params=[True, False], ids=["fused", "copy-then-multiply"])
def either_form(request):
    """Small problems are planned as copy-then-multiply; both forms are tested (keyword
    arguments for all_gather_matmul_tma_persistent)."""
    return {"fused": request.param}


@pytest.fixture(autouse=True)
def _release():
    yield
    from symm_mem_recipes import EmulatedSymmetricMemory as SM
    SM.release()


@pytest.mark.parametrize("M,N,K,ws,rank", [
    (2048, 256, 128, 8, 0),       # one K slab
    (2048, 400, 384, 8, 5),       # ragged last column tile
    (4096, 512, 1024, 8, 3),
    (2048, 272, 256, 4, 1),       # world size 4, two row tiles per comm block
    (1024, 256, 256, 8, 2),       # comm blocks of 128 rows: 128x128 tiles
    (1024, 144, 128, 8, 7),       # 128x128 tiles, ragged last column tile, one K slab
    (2048, 128, 1024, 8, 6),      # 128x128 tiles, eight K slabs
    (4096, 1280, 256, 8, 4),      # 256x128 tiles
    (8192, 1280, 128, 8, 1),      # 256x256 tiles, many of them
    (8192, 1280, 384, 8, 2),      # 256x256 tiles, three K slabs: the odd trip behind the K loop
    (4096, 1280, 640, 8, 7),      # 256x128 tiles, five K slabs
    (2048, 128, 896, 8, 3),       # 128x128 tiles, seven K slabs
])
def test_fp8_fused_parity(cuda, either_form, M, N, K, ws, rank):
    from symm_mem_recipes import all_gather_matmul_tma_persistent
    a_shard, h, shards, b, b_bits, a_out, c_out = _setup(M, N, K, ws, rank, cuda)
    ret = all_gather_matmul_tma_persistent(a_shard, b, a_out, c_out, None, **either_form)
    h.check_status()
    assert ret.data_ptr() == c_out.data_ptr()
    _check(_bits(c_out), O.ag_matmul_ref_fp8(shards, b_bits))
    assert np.array_equal(_bits(a_out), np.concatenate(shards))


def _random_shapes(n, seed):
    rng = np.random.default_rng(seed)
    shapes = []
    while len(shapes) < n:
        ws = int(rng.choice([2, 4, 5, 8]))
        comm = int(rng.choice([128, 256, 384, 512, 1024]))
        M = ws * comm
        N = 16 * int(rng.integers(1, 90))
        K = 128 * int(rng.integers(1, 9))
        shapes.append((M, N, K, ws, int(rng.integers(0, ws))))
    return shapes


@pytest.mark.parametrize("M,N,K,ws,rank", _random_shapes(10, seed=77))
def test_fp8_parity_random_shapes(cuda, either_form, M, N, K, ws, rank):
    from symm_mem_recipes import all_gather_matmul_tma_persistent
    a_shard, h, shards, b, b_bits, a_out, c_out = _setup(M, N, K, ws, rank, cuda)
    all_gather_matmul_tma_persistent(a_shard, b, a_out, c_out, None, **either_form)
    h.check_status()
    assert np.array_equal(_bits(a_out), np.concatenate(shards))
    _check(_bits(c_out), O.ag_matmul_ref_fp8(shards, b_bits))


def test_fp8_fused_entry_through_the_abi(cuda, lib):
    """The fused entry through the C ABI with e4m3fn operands: the codes of the Python call,
    gathered operand complete, state left zeroed."""
    from symm_mem_recipes import all_gather_matmul_tma_persistent
    M, N, K, ws, rank = 16384, 2048, 256, 8, 6
    a_shard, h, shards, b, b_bits, a_out, c_out = _setup(M, N, K, ws, rank, cuda)
    a_out.view(torch.uint8).zero_()
    c = torch.full_like(c_out.view(torch.uint8), 0x7F).view(torch.float8_e4m3fn)
    all_gather_matmul_tma_persistent(a_shard, b, a_out, c, None, fused=True)
    h.check_status()
    assert np.array_equal(_bits(a_out), np.concatenate(shards))
    want = _bits(c)
    _check(want, O.ag_matmul_ref_fp8(shards, b_bits))
    words = lib.smr_ag_matmul_fused_state_words(ws, 1)
    state = torch.zeros(words, dtype=torch.int32, device=cuda)
    a_out.view(torch.uint8).zero_()
    rc = lib.smr_ag_matmul_fused(a_shard.data_ptr(), a_out.data_ptr(), b.data_ptr(), c_out.data_ptr(),
                                 state.data_ptr(), h.buffer_ptrs_dev, 1, M, N, K, rank, ws, M // ws, 0,
                                 h.status.data_ptr(), torch.cuda.current_stream(cuda).cuda_stream)
    assert rc == 0
    h.check_status()
    assert state.cpu().tolist() == [0] * words
    assert np.array_equal(_bits(a_out), np.concatenate(shards))
    assert np.array_equal(_bits(c_out), want)


def test_fp8_saturation_and_exact_small_integers(cuda, either_form):
    """Operands of small integers: every product and sum is exact, so the result must
    equal the oracle bit for bit - including the entries beyond 448, which saturate."""
    from symm_mem_recipes import all_gather_matmul_tma_persistent
    M, N, K, ws = 2048, 256, 256, 8
    a_shard, h, shards, b, b_bits, a_out, c_out = _setup(M, N, K, ws, 2, cuda)
    rng = np.random.default_rng(1)
    vals = O.f32_to_fp8_e4m3fn(np.array([-4, -3, -2, -1, 0, 0, 0, 1, 2, 3, 4], dtype=np.float32))
    shards = [rng.choice(vals, size=(M // ws, K)).astype(np.uint8) for _ in range(ws)]
    for r in range(ws):
        h.get_buffer(r, (M // ws, K), torch.uint8).copy_(torch.from_numpy(shards[r]))
    b_bits = rng.choice(vals, size=(N, K)).astype(np.uint8)
    b = _t(b_bits).to(cuda)
    shards[0][0, :] = vals[-1]                     # 4 * 4 * 256 = 4096 -> saturates to 448
    shards[0][1, :] = vals[0]                      # -4 * 4 * 256 -> saturates to -448
    shards[0][2, 5] = 0x7F                         # one NaN in a row of A: the whole row of C is NaN
    b_bits[0, :] = vals[-1]
    h.get_buffer(0, (M // ws, K), torch.uint8).copy_(torch.from_numpy(shards[0]))
    b = _t(b_bits).to(cuda)
    all_gather_matmul_tma_persistent(a_shard, b, a_out, c_out, None, **either_form)
    h.check_status()
    want = O.ag_matmul_ref_fp8(shards, b_bits)
    got = _bits(c_out)
    assert got[0, 0] == 126 and want[0, 0] == 126
    assert got[1, 0] == 254 and want[1, 0] == 254
    assert np.all((got[2] & 0x7F) == 0x7F) and np.all((want[2] & 0x7F) == 0x7F)
    keep = np.arange(M) != 2                       # (a NaN's sign is not part of the contract)
    assert np.array_equal(got[keep], want[keep])


def test_fp8_mm_only_and_validation(cuda):
    from symm_mem_recipes import all_gather_matmul_tma_persistent
    M, N, K, ws = 2048, 256, 256, 8
    a_shard, h, shards, b, b_bits, a_out, c_out = _setup(M, N, K, ws, 0, cuda)
    a_out.view(torch.uint8).copy_(torch.from_numpy(np.concatenate(shards)))
    all_gather_matmul_tma_persistent(a_shard, b, a_out, c_out, None, mm_only=True)
    torch.cuda.synchronize()
    _check(_bits(c_out), O.ag_matmul_ref_fp8(shards, b_bits))
    with pytest.raises(AssertionError):             # K must be a multiple of 128
        all_gather_matmul_tma_persistent(a_shard[:, :192].contiguous(), b[:, :192].contiguous(),
                                         a_out[:, :192].contiguous(), c_out, None, mm_only=True)
    with pytest.raises(AssertionError):             # one dtype throughout
        all_gather_matmul_tma_persistent(a_shard, b, a_out, c_out.view(torch.uint8).to(torch.bfloat16), None)


def test_fp8_full_size_linearity(cuda):
    """M=16384 N=3584 K=8192 in e4m3fn: rows that touch every shard against the oracle,
    and all rows through C @ 1 == A @ (B^T @ 1) within the rounding of the cast."""
    from symm_mem_recipes import all_gather_matmul_tma_persistent
    M, N, K, ws = 16384, 3584, 8192, 8
    a_shard, h, shards, b, b_bits, a_out, c_out = _setup(M, N, K, ws, 0, cuda, std=0.05)
    all_gather_matmul_tma_persistent(a_shard, b, a_out, c_out, None)
    h.check_status()
    rows = sorted({s * 2048 + o for s in range(ws) for o in (0, 255, 256, 1023, 1500, 2047)})
    a_all = np.concatenate(shards)
    _check(_bits(c_out[rows]), O.ag_matmul_ref_fp8([a_all[rows]], b_bits))
    c = c_out.float()
    a = torch.cat([h.get_buffer(r, (M // ws, K), torch.float8_e4m3fn) for r in range(ws)]).float()
    rowsum = a @ b.float().sum(dim=0)
    # every entry is off by at most half an e4m3fn ulp (2^-4 relative); random walk over N entries
    tol = 8 * (N ** 0.5) * 2.0 ** -4 * float(c.pow(2).mean().sqrt()) + 1e-3
    assert torch.all((c.sum(dim=1) - rowsum).abs() <= tol)


@pytest.mark.parametrize("M,N,K", [(16384, 1792, 4096), (8192, 3584, 8192)])
def test_fp8_fused_launch_at_full_size_gathers_every_row(cuda, M, N, K):
    """The fused launch at sizes where its workgroups copy between two tiles with every register
    taken: the gathered operand equals the shards and the product equals the ungated launch's
    bit for bit.  (A register the compiler reloaded right behind one of the copy's assembly
    stores once changed what was stored: one row in sixteen of the last chunks, at the first of
    these shapes only.)"""
    from symm_mem_recipes import all_gather_matmul_tma_persistent
    ws = 8
    a_shard, h, shards, b, b_bits, a_out, c_out = _setup(M, N, K, ws, 0, cuda)
    want_a = np.concatenate(shards)
    for _ in range(3):
        a_out.view(torch.uint8).fill_(0x11)
        all_gather_matmul_tma_persistent(a_shard, b, a_out, c_out, None, fused=True)
        h.check_status()
        assert np.array_equal(_bits(a_out), want_a)
        fused_bits = _bits(c_out)
        c_out.view(torch.uint8).fill_(0x7F)
        all_gather_matmul_tma_persistent(a_shard, b, a_out, c_out, None, mm_only=True)
        h.check_status()
        assert np.array_equal(fused_bits, _bits(c_out))
