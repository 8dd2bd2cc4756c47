"""The gated GEMM behind flags that SOMEBODY ELSE raises: the reference's own choreography
(symm_mem_recipes/triton_all_gather_matmul.py:246-253, 318 - fresh zeroed `progress`, a
producer on another stream, a persistent GEMM that waits for each comm block's flag,
consumer side :170-174), through the C ABI (smr_all_gather_with_progress +
smr_ag_matmul(progress)) and through the Python entry point (fused="streams").

Checked: the product against the CPU oracle AND bit for bit against the ungated launch on
the gathered operand, the gathered operand against cat(shards), every flag up afterwards;
with the default flag wait (poll past the caches, no invalidate) and with the acquire fence
(smr_set_ag_matmul_acquire).  bf16 and e4m3fn."""
import numpy as np
import pytest
import torch

from oracle import oracle as O

pytestmark = pytest.mark.gpu


class _Bf16:
    dtype = torch.bfloat16
    elem = 2
    std = 0.02

    @staticmethod
    def bits(n, seed, std):
        return O.seeded_normal_bf16_bits(n, seed=seed, std=std)

    @staticmethod
    def to_t(bits):
        return torch.from_numpy(bits.view(np.int16).copy()).view(torch.bfloat16)

    @staticmethod
    def from_t(t):
        return t.contiguous().view(torch.int16).cpu().numpy().view(np.uint16)

    @staticmethod
    def ref(shards, b_bits):
        return O.ag_matmul_ref(shards, b_bits)

    @staticmethod
    def check(got_bits, want_bits):
        got = O.bf16_bits_to_f32(got_bits).astype(np.float64)
        want = O.bf16_bits_to_f32(want_bits).astype(np.float64)
        assert np.all(np.isfinite(got))
        rms = np.sqrt(np.mean(want ** 2))
        err = np.abs(got - want)
        # the path's tolerance: 1e-2 relative, with the result's scale for entries near zero
        assert np.all(err <= 1e-2 * np.abs(want) + 1e-2 * rms), float(err.max())


class _Fp8:
    dtype = torch.float8_e4m3fn
    elem = 1
    std = 0.25

    @staticmethod
    def bits(n, seed, std):
        return O.seeded_normal_fp8_bits(n, seed=seed, std=std)

    @staticmethod
    def to_t(bits):
        return torch.from_numpy(bits.copy()).view(torch.float8_e4m3fn)

    @staticmethod
    def from_t(t):
        return t.contiguous().view(torch.uint8).cpu().numpy()

    @staticmethod
    def ref(shards, b_bits):
        return O.ag_matmul_ref_fp8(shards, b_bits)

    @staticmethod
    def check(got, want):
        # codes as sign-magnitude integers: at most one code apart, >= 99.8 % identical
        assert not np.any((got & 0x7F) == 0x7F), "NaN in the result"
        key = lambda x: np.where(x & 0x80, -(x & 0x7F).astype(np.int32), (x & 0x7F).astype(np.int32))
        d = np.abs(key(got) - key(want))
        assert d.max() <= 1 and np.mean(d == 0) >= 0.998


KINDS = {"bf16": _Bf16, "e4m3fn": _Fp8}


def _setup(kind, M, N, K, ws, rank, cuda):
    from symm_mem_recipes import EmulatedSymmetricMemory as SM
    a_shard = SM.empty_strided_p2p((M // ws, K), (K, 1), kind.dtype, cuda, world_size=ws, rank=rank)
    h = SM.rendezvous(a_shard)
    shards = []
    for r in range(ws):
        bits = kind.bits(M // ws * K, r, kind.std).reshape(M // ws, K)
        h.get_buffer(r, (M // ws, K), kind.dtype).copy_(kind.to_t(bits))
        shards.append(bits)
    b_bits = kind.bits(N * K, 100, kind.std).reshape(N, K)
    b = kind.to_t(b_bits).to(cuda)
    a_out = torch.zeros(M * K * kind.elem, dtype=torch.uint8, device=cuda).view(kind.dtype).view(M, K)
    c_out = torch.zeros(M * N * kind.elem, dtype=torch.uint8, device=cuda).view(kind.dtype).view(M, N)
    return a_shard, h, shards, b, b_bits, a_out, c_out


@pytest.fixture(autouse=True)
def _release():
    yield
    from symm_mem_recipes import EmulatedSymmetricMemory as SM
    SM.release()


@pytest.fixture(params=[0, 1], ids=["flag-only", "acquire"])
def acquire_mode(request, lib):
    assert lib.smr_set_ag_matmul_acquire(request.param) == 0
    yield request.param
    lib.smr_set_ag_matmul_acquire(0)


def _gemm_entry(lib, kind):
    return lib.smr_ag_matmul_fp8 if kind.elem == 1 else lib.smr_ag_matmul


def _ungated_bits(lib, kind, a_shard, h, shards, b, M, N, K, ws, rank, splits, cuda):
    """The ungated launch on an operand gathered by torch: the bits the gated launch must give."""
    a_ref = kind.to_t(np.concatenate(shards)).to(cuda)
    c_ref = torch.zeros(M * N * kind.elem, dtype=torch.uint8, device=cuda).view(kind.dtype).view(M, N)
    rc = _gemm_entry(lib, kind)(a_shard.data_ptr(), a_ref.data_ptr(), b.data_ptr(), c_ref.data_ptr(), None, M, N, K,
                                rank, ws, M // ws // splits, 0, h.status.data_ptr(),
                                torch.cuda.current_stream(cuda).cuda_stream)
    assert rc == 0, lib.smr_last_error_string()
    h.check_status()
    return kind.from_t(c_ref)


@pytest.mark.parametrize("kind_name", ["bf16", "e4m3fn"])
@pytest.mark.parametrize("M,N,K,rank,splits", [
    (8192, 1024, 1024, 0, 1),      # 256x256 tiles, four K slab pairs...
    (8192, 1024, 1024, 5, 2),      # ... two flags per rank
    (4096, 384, 256, 5, 1),        # narrow: 256x128 tiles, ragged column tile
    (2048, 256, 384, 0, 2),        # comm blocks of 128 rows: 128x128 tiles
])
def test_gated_gemm_behind_the_stand_alone_producer(cuda, lib, acquire_mode, kind_name, M, N, K, rank, splits):
    """Same stream, no co-residency needed: smr_all_gather_with_progress into a_out + progress,
    then smr_ag_matmul(progress) behind it.  Every non-local tile takes the `wait_flag_set`
    branch with flags that a different kernel raised."""
    kind, ws = KINDS[kind_name], 8
    a_shard, h, shards, b, b_bits, a_out, c_out = _setup(kind, M, N, K, ws, rank, cuda)
    want_bits = _ungated_bits(lib, kind, a_shard, h, shards, b, M, N, K, ws, rank, splits, cuda)
    chunks = ws * splits
    flags = torch.zeros(2 * chunks, dtype=torch.int32, device=cuda)
    progress, counters = flags[:chunks], flags[chunks:]
    st = torch.cuda.current_stream(cuda).cuda_stream
    print(f"producer then gated GEMM: {kind_name} M {M} N {N} K {K} rank {rank} splits {splits} acquire {acquire_mode}", flush=True)
    rc = lib.smr_all_gather_with_progress(h.buffer_ptrs_dev, a_out.data_ptr(), progress.data_ptr(), counters.data_ptr(),
                                          rank, ws, (M // ws) * K * kind.elem, splits, 16, st)
    assert rc == 0, lib.smr_last_error_string()
    rc = _gemm_entry(lib, kind)(a_shard.data_ptr(), a_out.data_ptr(), b.data_ptr(), c_out.data_ptr(),
                                progress.data_ptr(), M, N, K, rank, ws, M // ws // splits, 0, h.status.data_ptr(), st)
    assert rc == 0, lib.smr_last_error_string()
    h.check_status()
    assert progress.cpu().tolist() == [1] * chunks
    assert np.array_equal(kind.from_t(a_out), np.concatenate(shards))
    got = kind.from_t(c_out)
    assert np.array_equal(got, want_bits)
    kind.check(got, kind.ref(shards, b_bits))


@pytest.mark.parametrize("beside", [False, True], ids=["producer-on-its-own-CUs", "producer-beside-the-GEMM"])
@pytest.mark.parametrize("kind_name,M,N,K,rank,splits", [
    ("bf16", 8192, 1024, 1024, 0, 1), ("bf16", 8192, 1024, 1024, 5, 2),
    ("e4m3fn", 8192, 1024, 1024, 5, 1), ("e4m3fn", 8192, 1280, 512, 0, 2),
    ("bf16", 16384, 3584, 8192, 0, 1),            # the full-size problem
])
def test_gated_gemm_beside_the_producer_on_another_stream(cuda, lib, acquire_mode, beside, kind_name, M, N, K, rank, splits):
    """The reference's choreography through the C ABI: progress zeroed, the producer on a side
    stream, smr_ag_matmul(progress) on the current stream, join.  Either the GEMM's grid leaves
    compute units free for the producer (smr_all_gather_with_progress, whole_gpu = 0), or the
    producer's workgroups fit beside the GEMM's on the same compute units and the GEMM takes
    them all (smr_all_gather_beside, whole_gpu = 1); the two kernels run side by side whichever
    is dispatched first."""
    import ctypes
    kind, ws = KINDS[kind_name], 8
    a_shard, h, shards, b, b_bits, a_out, c_out = _setup(kind, M, N, K, ws, rank, cuda)
    want_bits = _ungated_bits(lib, kind, a_shard, h, shards, b, M, N, K, ws, rank, splits, cuda)
    chunks = ws * splits
    plan = (ctypes.c_int32 * 5)()
    planner = lib.smr_ag_matmul_plan_fp8 if kind.elem == 1 else lib.smr_ag_matmul_plan
    assert planner(M, N, K, ws, M // ws // splits, plan) == 0
    flags = torch.zeros(2 * chunks, dtype=torch.int32, device=cuda)
    progress, counters = flags[:chunks], flags[chunks:]
    current = torch.cuda.current_stream(cuda)
    side = torch.cuda.Stream(cuda)
    side.wait_stream(current)
    print(f"producer beside gated GEMM: {kind_name} M {M} N {N} K {K} rank {rank} splits {splits} "
          f"acquire {acquire_mode} beside {beside} grid {plan[0]} + {plan[1]}", flush=True)
    producer = lib.smr_all_gather_beside if beside else lib.smr_all_gather_with_progress
    # (the producer beside the GEMM on the timetable of the planner's estimate, and in the second
    # parameter set on one four times as long: then it is the GEMM that waits, which must not matter)
    timetable = []
    if beside:
        pace = (ctypes.c_int32 * 2)()
        assert lib.smr_ag_matmul_pace(M, N, K, ws, M // ws // splits, kind.elem, pace) == 0
        timetable = [max(pace[0], 10) * 4, 1] if splits == 2 else [pace[0], pace[1]]
    rc = producer(h.buffer_ptrs_dev, a_out.data_ptr(), progress.data_ptr(), counters.data_ptr(),
                  rank, ws, (M // ws) * K * kind.elem, splits, 0 if beside else plan[1], *timetable, side.cuda_stream)
    assert rc == 0, lib.smr_last_error_string()
    rc = _gemm_entry(lib, kind)(a_shard.data_ptr(), a_out.data_ptr(), b.data_ptr(), c_out.data_ptr(),
                                progress.data_ptr(), M, N, K, rank, ws, M // ws // splits, int(beside),
                                h.status.data_ptr(), current.cuda_stream)
    assert rc == 0, lib.smr_last_error_string()
    current.wait_stream(side)
    h.check_status()
    assert progress.cpu().tolist() == [1] * chunks
    got = kind.from_t(c_out)
    assert np.array_equal(got, want_bits)
    if M * K <= 1 << 24:
        assert np.array_equal(kind.from_t(a_out), np.concatenate(shards))
        kind.check(got, kind.ref(shards, b_bits))
    else:                                            # the full product costs a TFLOP on the CPU: sampled rows
        rows = sorted({s * (M // ws) + o for s in range(ws) for o in (0, 255, 256, 1023, 2047)})
        a_all = np.concatenate(shards)
        assert np.array_equal(kind.from_t(a_out[rows]), a_all[rows])
        assert torch.equal(a_out.view(torch.int16), kind.to_t(a_all).to(cuda).view(torch.int16))
        kind.check(got[rows], kind.ref([a_all[rows]], b_bits))


@pytest.mark.parametrize("rank,splits", [(0, 1), (3, 2)])
def test_flags_raised_one_by_one_with_stream_write_value32(cuda, lib, acquire_mode, rank, splits):
    """The reference's producer as it is written (triton_all_gather_matmul.py:41-55): per chunk a
    copy_ into the gathered operand and a stream-ordered 32-bit write that raises its flag, in the
    reference's order, on the backend stream; the GEMM on the current stream waits flag by flag."""
    from symm_mem_recipes import _get_backend_stream
    kind, ws = _Bf16, 8
    M, N, K = 8192, 1024, 1024
    a_shard, h, shards, b, b_bits, a_out, c_out = _setup(kind, M, N, K, ws, rank, cuda)
    want_bits = _ungated_bits(lib, kind, a_shard, h, shards, b, M, N, K, ws, rank, splits, cuda)
    chunks = ws * splits
    progress = torch.zeros(chunks, dtype=torch.int32, device=cuda)
    current = torch.cuda.current_stream(cuda)
    backend = _get_backend_stream()
    backend.wait_stream(current)
    rows = M // ws // splits
    out_chunks = a_out.chunk(chunks)
    with torch.cuda.stream(backend):
        for step in range(ws):
            src_rank = (rank + step + 1) % ws
            src = h.get_buffer(src_rank, (M // ws, K), kind.dtype)
            for split in range(splits):
                idx = src_rank * splits + split
                out_chunks[idx].copy_(src[split * rows:(split + 1) * rows])
                h.stream_write_value32(progress.data_ptr() + idx * progress.element_size(), 1)
    rc = lib.smr_ag_matmul(a_shard.data_ptr(), a_out.data_ptr(), b.data_ptr(), c_out.data_ptr(), progress.data_ptr(),
                           M, N, K, rank, ws, rows, 0, h.status.data_ptr(), current.cuda_stream)
    assert rc == 0, lib.smr_last_error_string()
    current.wait_stream(backend)
    h.check_status()
    assert progress.cpu().tolist() == [1] * chunks
    assert np.array_equal(kind.from_t(a_out), np.concatenate(shards))
    assert np.array_equal(kind.from_t(c_out), want_bits)


@pytest.mark.parametrize("M,N,K", [(8192, 1024, 1024), (16384, 2048, 256)])
def test_streams_form_reads_fresh_rows_when_buffers_are_reused(cuda, acquire_mode, M, N, K):
    """The same gathered buffer, the same output and new shard contents call after call in the
    two-stream form, with no host synchronisation in between: a tile must never be computed from
    rows that a cache kept from the call before (the gathered operand of these shapes fits the L2s)."""
    from symm_mem_recipes import all_gather_matmul_tma_persistent
    kind, ws, rank = _Bf16, 8, 4
    a_shard, h, shards, b, b_bits, a_out, c_out = _setup(kind, M, N, K, ws, rank, cuda)
    rows = M // ws
    versions = []
    for v in range(4):
        bits = [kind.bits(rows * K, 1000 * v + r, kind.std).reshape(rows, K) for r in range(ws)]
        versions.append((bits, [kind.to_t(x).to(cuda) for x in bits]))
    outs = []
    for bits, dev_bits in versions:
        for r in range(ws):
            h.get_buffer(r, (rows, K), kind.dtype).copy_(dev_bits[r])
        all_gather_matmul_tma_persistent(a_shard, b, a_out, c_out, None, fused="streams")
        outs.append((c_out.clone(), a_out.clone()))
    torch.cuda.synchronize()
    h.check_status()
    for (bits, _), (c, a) in zip(versions, outs):
        assert np.array_equal(kind.from_t(a), np.concatenate(bits))
        kind.check(kind.from_t(c), kind.ref(bits, b_bits))


@pytest.mark.parametrize("kind_name,splits", [("bf16", 1), ("bf16", 2), ("e4m3fn", 1)])
def test_streams_form_of_the_python_entry_point(cuda, kind_name, splits):
    """all_gather_matmul_tma_persistent(fused="streams") gives the bits of the one-launch form."""
    from symm_mem_recipes import all_gather_matmul_tma_persistent
    kind, ws, rank = KINDS[kind_name], 8, 6
    M, N, K = 8192, 1280, 512
    a_shard, h, shards, b, b_bits, a_out, c_out = _setup(kind, M, N, K, ws, rank, cuda)
    all_gather_matmul_tma_persistent(a_shard, b, a_out, c_out, None, splits_per_rank=splits, fused=True)
    h.check_status()
    want = kind.from_t(c_out)
    for _ in range(3):
        a_out.view(torch.uint8).zero_()
        c_out.view(torch.uint8).zero_()
        ret = all_gather_matmul_tma_persistent(a_shard, b, a_out, c_out, None, splits_per_rank=splits, fused="streams")
        h.check_status()
        assert ret.data_ptr() == c_out.data_ptr()
        assert np.array_equal(kind.from_t(a_out), np.concatenate(shards))
        assert np.array_equal(kind.from_t(c_out), want)
    kind.check(want, kind.ref(shards, b_bits))
