"""GPU parity of the all-gather producer and the flag-gated GEMM against the CPU
oracle (cat + fp32 matmul, rounded to bf16).  Tolerance, as stated for this path:
1e-2 relative; checked elementwise as |got - want| <= 1e-2 * |want| + 1e-2 * rms(want)
(the second term covers entries near zero, where bf16 rounding of either side
dominates), and additionally 99.9 % of entries within 1 bf16 ulp."""
import numpy as np
import pytest
import torch

from oracle import oracle as O

pytestmark = pytest.mark.gpu


def _bits_t(bits):
    return torch.from_numpy(bits.view(np.int16).copy()).view(torch.bfloat16)


def _t_bits(t):
    return t.contiguous().view(torch.int16).cpu().numpy().view(np.uint16)


def _setup(M, N, K, ws, rank, cuda, std=0.02):
    from symm_mem_recipes import EmulatedSymmetricMemory as SM
    a_shard = SM.empty_strided_p2p((M // ws, K), (K, 1), torch.bfloat16, cuda, world_size=ws, rank=rank)
    h = SM.rendezvous(a_shard)
    shards = []
    for r in range(ws):
        bits = O.seeded_normal_bf16_bits(M // ws * K, seed=r, std=std).reshape(M // ws, K)
        h.get_buffer(r, (M // ws, K), torch.bfloat16).copy_(_bits_t(bits))
        shards.append(bits)
    b_bits = O.seeded_normal_bf16_bits(N * K, seed=100, std=std).reshape(N, K)
    b = _bits_t(b_bits).to(cuda)
    a_out = torch.full((M, K), float("nan"), dtype=torch.bfloat16, device=cuda)
    c_out = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device=cuda)
    return a_shard, h, shards, b, b_bits, a_out, c_out


def _check(got_bits, want_bits):
    got = O.bf16_bits_to_f32(got_bits).astype(np.float64)
    want = O.bf16_bits_to_f32(want_bits).astype(np.float64)
    assert np.all(np.isfinite(got))
    rms = np.sqrt(np.mean(want ** 2))
    err = np.abs(got - want)
    assert np.all(err <= 1e-2 * np.abs(want) + 1e-2 * rms), float(err.max())
    ulp = np.maximum(np.abs(want), 2.0 ** -126) * 2.0 ** -7
    assert np.mean(err <= ulp) >= 0.999


@pytest.fixture
def force_fused():
    """Small problems are planned as copy-then-multiply; the tests of the flag-gated
    launch force it (keyword arguments for all_gather_matmul_tma_persistent)."""
    return {"fused": True}


@pytest.fixture(params=[True, False], ids=["fused", "copy-then-multiply"])
def either_form(request):
    return {"fused": request.param}


@pytest.fixture(autouse=True)
def _release():
    yield
    from symm_mem_recipes import EmulatedSymmetricMemory as SM
    SM.release()


@pytest.mark.parametrize("rank,splits", [(0, 1), (5, 1), (2, 2)])
def test_all_gather_with_progress(cuda, rank, splits):
    from symm_mem_recipes import all_gather_with_progress
    ws, rows, K = 8, 96, 200
    a_shard, h, shards, *_ = _setup(ws * rows, 8, K, ws, rank, cuda)
    out = torch.zeros(ws * rows, K, dtype=torch.bfloat16, device=cuda)
    progress = torch.zeros(ws * splits, dtype=torch.int32, device=cuda)
    all_gather_with_progress(out, a_shard, progress, splits)
    torch.cuda.synchronize()
    want, prog, _ = O.all_gather_ref(shards, rank, splits)
    assert np.array_equal(_t_bits(out), want)
    assert progress.cpu().tolist() == prog.tolist()


@pytest.mark.parametrize("rank,splits", [(0, 1), (5, 2), (7, 4)])
def test_flags_go_up_in_the_reference_order(cuda, lib, rank, splits):
    """The order in which the producer raises the progress flags
    (triton_all_gather_matmul.py:43-44: sources rank+1, ..., rank+ws-1, rank; splits of a
    source in order), read from the time stamps it leaves in the trace buffer.  (In the
    fused launch only the walk of the copy-only workgroups is fixed: a GEMM workgroup that
    finds its chunk missing copies at it, so a chunk can be complete out of turn.)"""
    from symm_mem_recipes import all_gather_with_progress
    ws, rows, K = 8, 2048, 1024                         # 4 MiB per rank: a chunk takes microseconds, the clock ticks every 10 ns
    a_shard, h, shards, b, b_bits, a_out, c_out = _setup(ws * rows, 8, K, ws, rank, cuda)
    words = 64 + 256 * 16 * 4
    trace = torch.zeros(words, dtype=torch.int64, device=cuda)
    chunks = ws * splits
    try:
        assert lib.smr_set_trace_buffer(trace.data_ptr(), words) == 0
        progress = torch.zeros(chunks, dtype=torch.int32, device=cuda)
        all_gather_with_progress(a_out, a_shard, progress, splits, num_workgroups=4)
        torch.cuda.synchronize()
        h.check_status()
    finally:
        lib.smr_set_trace_buffer(None, 0)
    stamps = trace[:chunks].cpu().tolist()
    assert all(t > 0 for t in stamps), stamps
    order = sorted(range(chunks), key=lambda i: stamps[i])
    assert order == list(O.all_gather_ref(shards, rank, splits)[2]), order
    assert progress.cpu().tolist() == [1] * chunks
    assert np.array_equal(_t_bits(a_out), np.concatenate(shards))


@pytest.mark.parametrize("ws,rows,K,splits,wgs", [(8, 96, 200, 1, 3), (8, 96, 200, 2, 256), (3, 64, 72, 4, 1),
                                                 (8, 8, 8, 1, 256), (8, 512, 4096, 4, 256)])
def test_all_gather_at_once(cuda, lib, ws, rows, K, splits, wgs):
    """All chunks copied together (the copy a GEMM is queued behind): the same gathered
    operand, flags and zeroed counters as the chunk-by-chunk producer leaves."""
    rank = ws - 1
    a_shard, h, shards, *_ = _setup(ws * rows, 8, K, ws, rank, cuda)
    out = torch.zeros(ws * rows, K, dtype=torch.bfloat16, device=cuda)
    state = torch.zeros(2 * ws * splits, dtype=torch.int32, device=cuda)
    progress, counters = state[:ws * splits], state[ws * splits:]
    for _ in range(2):                                   # the counters are left ready for the next call
        out.zero_()
        progress.zero_()
        rc = lib.smr_all_gather_at_once(h.buffer_ptrs_dev, out.data_ptr(), progress.data_ptr(),
                                        counters.data_ptr(), rank, ws, rows * K * 2, splits, wgs,
                                        torch.cuda.current_stream(cuda).cuda_stream)
        assert rc == 0
        torch.cuda.synchronize()
        want, prog, _ = O.all_gather_ref(shards, rank, splits)
        assert np.array_equal(_t_bits(out), want)
        assert progress.cpu().tolist() == prog.tolist()
        assert counters.cpu().tolist() == [0] * (ws * splits)


@pytest.mark.parametrize("M,N,K,ws,rank", [
    (1024, 256, 256, 8, 0),      # 128x128 tiles
    (1024, 136, 64, 8, 6),       # ragged last column tile, single K step
    (2048, 384, 512, 8, 3),      # 256x256 tiles with a half-empty column tile
    (2048, 128, 1024, 8, 7),     # 256x128 tiles
    (1024, 512, 320, 4, 1),      # world size 4
])
def test_fused_parity_small(cuda, either_form, M, N, K, ws, rank):
    from symm_mem_recipes import all_gather_matmul_tma_persistent, all_gather_matmul
    a_shard, h, shards, b, b_bits, a_out, c_out = _setup(M, N, K, ws, rank, cuda)
    configs = {"BLOCK_SIZE_M": 128, "BLOCK_SIZE_N": 128, "BLOCK_SIZE_K": 64, "GROUP_SIZE_M": 1,
               "num_stages": 3, "num_warps": 8}
    ret = all_gather_matmul_tma_persistent(a_shard, b, a_out, c_out, configs, **either_form)
    h.check_status()
    assert ret.data_ptr() == c_out.data_ptr()
    want = O.ag_matmul_ref(shards, b_bits)
    _check(_t_bits(c_out), want)
    # the gathered operand is complete too
    assert np.array_equal(_t_bits(a_out), np.concatenate(shards))
    # the reference's own check: fused == all-gather + library matmul (allclose)
    c0 = all_gather_matmul(a_shard, b.T)
    assert torch.allclose(c0.float(), c_out.float(), rtol=2e-2, atol=1e-3)


@pytest.mark.parametrize("M,N,K,ws,rank,splits", [
    (2048, 256, 256, 8, 3, 2),       # comm blocks of 128 rows: 128x128 tiles
    (4096, 512, 128, 8, 6, 2),       # comm blocks of 256 rows: 256x256 tiles, 16 flags
    (4096, 384, 192, 4, 1, 4),       # world size 4, four flags per rank
])
def test_fused_parity_splits_per_rank(cuda, either_form, M, N, K, ws, rank, splits):
    """Finer flags (triton_all_gather_matmul.py:24,41-49): every rank's shard arrives in
    `splits` chunks with a flag each, and a tile waits for the chunk its rows are in."""
    from symm_mem_recipes import all_gather_matmul_tma_persistent
    a_shard, h, shards, b, b_bits, a_out, c_out = _setup(M, N, K, ws, rank, cuda)
    a_out.zero_()
    all_gather_matmul_tma_persistent(a_shard, b, a_out, c_out, None, splits_per_rank=splits, **either_form)
    h.check_status()
    _check(_t_bits(c_out), O.ag_matmul_ref(shards, b_bits))
    assert np.array_equal(_t_bits(a_out), np.concatenate(shards))


def test_fused_back_to_back_calls_are_identical(cuda, either_form):
    """Twenty fused launches in a row without a host synchronisation in between, the
    gathered operand wiped before each: flags, arrival counters and the two streams
    must hand over cleanly from one call to the next, and the result is deterministic."""
    from symm_mem_recipes import all_gather_matmul_tma_persistent
    M, N, K, ws, rank = 8192, 1024, 1024, 8, 6
    a_shard, h, shards, b, b_bits, a_out, c_out = _setup(M, N, K, ws, rank, cuda)
    outs = []
    for i in range(20):
        a_out.zero_()
        c = torch.empty_like(c_out)
        all_gather_matmul_tma_persistent(a_shard, b, a_out, c, None, **either_form)
        outs.append(c)
    torch.cuda.synchronize()
    h.check_status()
    _check(_t_bits(outs[0]), O.ag_matmul_ref(shards, b_bits))
    assert np.array_equal(_t_bits(a_out), np.concatenate(shards))
    for c in outs[1:]:
        assert torch.equal(c.view(torch.int16), outs[0].view(torch.int16))


def test_copy_then_multiply_matches_fused(cuda, lib):
    """A GEMM too short to hide the copy behind is planned as copy-then-multiply
    (M=2048 N=4096 K=2048 is); the planned form and both forced forms give the oracle's
    product and one another's bits, with the gathered operand complete in each."""
    import ctypes
    import importlib
    agm = importlib.import_module("symm_mem_recipes.all_gather_matmul")
    M, N, K, ws, rank = 2048, 4096, 2048, 8, 3
    plan = (ctypes.c_int32 * 5)()
    assert lib.smr_ag_matmul_plan(M, N, K, ws, M // ws, plan) == 0 and plan[4] == 1
    a_shard, h, shards, b, b_bits, a_out, c_out = _setup(M, N, K, ws, rank, cuda)
    want = O.ag_matmul_ref(shards, b_bits)
    outs = []
    for fused in (None, True, False):
        a_out.zero_()
        c = torch.full_like(c_out, float("nan"))
        agm.all_gather_matmul_tma_persistent(a_shard, b, a_out, c, None, fused=fused)
        h.check_status()
        assert np.array_equal(_t_bits(a_out), np.concatenate(shards))
        _check(_t_bits(c), want)
        outs.append(c)
    assert torch.equal(outs[0].view(torch.int16), outs[1].view(torch.int16))
    assert torch.equal(outs[0].view(torch.int16), outs[2].view(torch.int16))


@pytest.mark.parametrize("M,N,K", [(8192, 1024, 1024), (4096, 1792, 4096)])
def test_fused_launch_replays_from_a_graph(cuda, either_form, M, N, K):
    """The whole call captured into a HIP graph (kernel nodes only) and replayed: every
    replay, with eager work and synchronisations in between, gives the eager result, for the
    fused form (one launch whose flags the kernel itself leaves zeroed) and for
    copy-then-multiply."""
    from symm_mem_recipes import all_gather_matmul_tma_persistent
    ws, rank = 8, 2
    a_shard, h, shards, b, b_bits, a_out, c_out = _setup(M, N, K, ws, rank, cuda)
    all_gather_matmul_tma_persistent(a_shard, b, a_out, c_out, None, **either_form)          # eager: the expected bits
    torch.cuda.synchronize()
    h.check_status()
    want_c, want_a = c_out.clone(), a_out.clone()
    _check(_t_bits(want_c)[:64], O.ag_matmul_ref([shards[0][:64]], b_bits))
    side = torch.cuda.Stream(cuda)
    side.wait_stream(torch.cuda.current_stream(cuda))
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            all_gather_matmul_tma_persistent(a_shard, b, a_out, c_out, None, **either_form)
    torch.cuda.current_stream(cuda).wait_stream(side)
    for replay in range(4):
        a_out.zero_()
        c_out.fill_(float("nan"))
        scratch = torch.randn(1 << 20, device=cuda).sum()                      # unrelated eager work
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        h.check_status()
        assert torch.equal(c_out.view(torch.int16), want_c.view(torch.int16)), replay
        assert torch.equal(a_out.view(torch.int16), want_a.view(torch.int16)), replay
        del scratch
    del graph


@pytest.mark.parametrize("producers", [1, 8, 64])
def test_fused_entry_through_the_abi(cuda, lib, producers):
    """smr_ag_matmul_fused called directly, twice on one state array that is zeroed once:
    product as the oracle's, gathered operand complete, and every word of the state (flags,
    tickets, counters) zero again after each launch."""
    M, N, K, ws, rank, splits = 4096, 512, 256, 8, 3, 2
    a_shard, h, shards, b, b_bits, a_out, c_out = _setup(M, N, K, ws, rank, cuda)
    words = lib.smr_ag_matmul_fused_state_words(ws, splits)
    assert words == 3 * ws * splits + 1
    state = torch.zeros(words, dtype=torch.int32, device=cuda)
    want = O.ag_matmul_ref(shards, b_bits)
    for call in range(2):
        a_out.zero_()
        c_out.fill_(float("nan"))
        rc = lib.smr_ag_matmul_fused(a_shard.data_ptr(), a_out.data_ptr(), b.data_ptr(), c_out.data_ptr(),
                                     state.data_ptr(), h.buffer_ptrs_dev, 2, M, N, K, rank, ws, M // ws // splits,
                                     producers, h.status.data_ptr(), torch.cuda.current_stream(cuda).cuda_stream)
        assert rc == 0, lib.smr_last_error_string()
        h.check_status()
        assert state.cpu().tolist() == [0] * words, call
        assert np.array_equal(_t_bits(a_out), np.concatenate(shards))
        _check(_t_bits(c_out), want)
    bad = lib.smr_ag_matmul_fused
    args = (a_shard.data_ptr(), a_out.data_ptr(), b.data_ptr(), c_out.data_ptr())
    assert bad(*args, None, h.buffer_ptrs_dev, 2, M, N, K, rank, ws, M // ws, 0, None, None) == -1
    assert bad(*args, state.data_ptr(), None, 2, M, N, K, rank, ws, M // ws, 0, None, None) == -1
    assert bad(*args, state.data_ptr(), h.buffer_ptrs_dev, 4, M, N, K, rank, ws, M // ws, 0, None, None) == -1
    assert bad(*args, state.data_ptr(), h.buffer_ptrs_dev, 2, M, N, K, rank, ws, M // ws, -3, None, None) == -1


def test_fused_launch_needs_no_second_stream(cuda, lib):
    """The fused call issues exactly one kernel on the current stream: run on a side stream
    with nothing else in flight, with the copy-only workgroups taken away altogether (the
    GEMM's workgroups then do all the copying themselves), it still completes and is right."""
    from symm_mem_recipes import all_gather_matmul_tma_persistent
    M, N, K, ws, rank = 8192, 1024, 512, 8, 2
    a_shard, h, shards, b, b_bits, a_out, c_out = _setup(M, N, K, ws, rank, cuda)
    want = O.ag_matmul_ref(shards, b_bits)
    side = torch.cuda.Stream(cuda)
    side.wait_stream(torch.cuda.current_stream(cuda))
    with torch.cuda.stream(side):
        a_out.zero_()
        all_gather_matmul_tma_persistent(a_shard, b, a_out, c_out, None, fused=True, check=True)
    side.synchronize()
    _check(_t_bits(c_out), want)
    assert np.array_equal(_t_bits(a_out), np.concatenate(shards))
    # no copy-only workgroup at all: smr_ag_matmul_fused with a grid that leaves no room for them
    try:
        assert lib.smr_set_ag_matmul_grid_limit(0) == 0
        words = lib.smr_ag_matmul_fused_state_words(ws, 1)
        state = torch.zeros(words, dtype=torch.int32, device=cuda)
        a_out.zero_()
        c_out.fill_(float("nan"))
        # one copy-only workgroup: the waiters do most of the copying
        rc = lib.smr_ag_matmul_fused(a_shard.data_ptr(), a_out.data_ptr(), b.data_ptr(), c_out.data_ptr(),
                                     state.data_ptr(), h.buffer_ptrs_dev, 2, M, N, K, rank, ws, M // ws, 1,
                                     h.status.data_ptr(), torch.cuda.current_stream(cuda).cuda_stream)
        assert rc == 0
        h.check_status()
    finally:
        lib.smr_set_ag_matmul_grid_limit(0)
    _check(_t_bits(c_out), want)
    assert np.array_equal(_t_bits(a_out), np.concatenate(shards))
    assert state.cpu().tolist() == [0] * words


@pytest.fixture(params=[0, 1], ids=["flag-only", "acquire"])
def acquire_mode(request, lib):
    assert lib.smr_set_ag_matmul_acquire(request.param) == 0
    yield request.param
    lib.smr_set_ag_matmul_acquire(0)


@pytest.mark.parametrize("M,N,K", [(8192, 1024, 1024), (16384, 2048, 256)])
def test_fused_reads_fresh_rows_when_buffers_are_reused(cuda, either_form, acquire_mode, M, N, K):
    """The same gathered buffer, the same output and new shard contents call after call,
    with no host synchronisation in between: a tile must never be computed from rows that
    a cache kept from the call before (the gathered operand of these shapes fits the L2s)."""
    from symm_mem_recipes import all_gather_matmul_tma_persistent
    ws, rank = 8, 4
    a_shard, h, shards, b, b_bits, a_out, c_out = _setup(M, N, K, ws, rank, cuda)
    rows = M // ws
    versions = []
    for v in range(4):
        bits = [O.seeded_normal_bf16_bits(rows * K, seed=1000 * v + r, std=0.02).reshape(rows, K) for r in range(ws)]
        versions.append((bits, [_bits_t(x).to(cuda) for x in bits]))
    outs = []
    for bits, dev_bits in versions:
        for r in range(ws):
            h.get_buffer(r, (rows, K), torch.bfloat16).copy_(dev_bits[r])
        all_gather_matmul_tma_persistent(a_shard, b, a_out, c_out, None, **either_form)
        outs.append((c_out.clone(), a_out.clone()))
    torch.cuda.synchronize()
    h.check_status()
    for (bits, _), (c, a) in zip(versions, outs):
        assert np.array_equal(_t_bits(a), np.concatenate(bits))
        _check(_t_bits(c), O.ag_matmul_ref(bits, b_bits))


def _random_shapes(n, seed):
    rng = np.random.default_rng(seed)
    shapes = []
    while len(shapes) < n:
        ws = int(rng.choice([2, 3, 4, 5, 8]))
        splits = int(rng.choice([1, 1, 2, 3]))
        comm = int(rng.choice([128, 256, 384, 512, 768, 1024]))
        M = ws * splits * comm
        N = 8 * int(rng.integers(1, 190))
        K = 64 * int(rng.integers(1, 17))
        if M * N * K > 8e9:
            continue
        shapes.append((M, N, K, ws, int(rng.integers(0, ws)), splits))
    return shapes


@pytest.mark.parametrize("M,N,K,ws,rank,splits", _random_shapes(14, seed=2024))
def test_fused_parity_random_shapes(cuda, either_form, M, N, K, ws, rank, splits):
    """Shapes drawn at random from what the kernel accepts (every world size, ragged column
    tiles, one to sixteen K slabs, one to three flags per rank): product and gathered operand
    against the oracle in both forms of the launch."""
    from symm_mem_recipes import all_gather_matmul_tma_persistent
    a_shard, h, shards, b, b_bits, a_out, c_out = _setup(M, N, K, ws, rank, cuda)
    a_out.zero_()
    all_gather_matmul_tma_persistent(a_shard, b, a_out, c_out, None, splits_per_rank=splits, **either_form)
    h.check_status()
    assert np.array_equal(_t_bits(a_out), np.concatenate(shards))
    _check(_t_bits(c_out), O.ag_matmul_ref(shards, b_bits))


def test_mm_only_is_ungated(cuda, monkeypatch):
    """mm_only multiplies what the buffers already hold, as rank 0, with no flags
    (triton_all_gather_matmul.py:222-224,246-247)."""
    from symm_mem_recipes import all_gather_matmul_tma_persistent
    monkeypatch.setenv("WORLD_SIZE", "8")
    M, N, K, ws = 2048, 256, 256, 8
    a_shard, h, shards, b, b_bits, a_out, c_out = _setup(M, N, K, ws, 0, cuda)
    a_out.copy_(_bits_t(np.concatenate(shards)))
    a_out[: M // ws].fill_(float("nan"))          # rank 0's rows must come from a_shard
    all_gather_matmul_tma_persistent(a_shard, b, a_out, c_out, None, mm_only=True)
    torch.cuda.synchronize()
    _check(_t_bits(c_out), O.ag_matmul_ref(shards, b_bits))


def test_gemm_waits_for_flags(cuda, lib):
    """With a progress array that is never set the kernel must report a wait
    timeout (bounded spin forced from the host) instead of reading early."""
    from symm_mem_recipes import _lib
    M, N, K, ws = 1024, 128, 64, 8
    a_shard, h, shards, b, b_bits, a_out, c_out = _setup(M, N, K, ws, 0, cuda)
    progress = torch.zeros(ws, dtype=torch.int32, device=cuda)
    old = lib.smr_get_spin_timeout_us()
    lib.smr_set_spin_timeout_us(500)
    try:
        rc = lib.smr_ag_matmul(a_shard.data_ptr(), a_out.data_ptr(), b.data_ptr(), c_out.data_ptr(),
                               progress.data_ptr(), M, N, K, 0, ws, M // ws, 0, h.status.data_ptr(),
                               torch.cuda.current_stream().cuda_stream)
        assert rc == 0
        with pytest.raises(_lib.SmrError, match="wait_signal timed out"):
            h.check_status()
    finally:
        lib.smr_set_spin_timeout_us(old)


def test_validation(cuda):
    from symm_mem_recipes import all_gather_matmul_tma_persistent
    a_shard, h, shards, b, b_bits, a_out, c_out = _setup(1024, 128, 64, 8, 0, cuda)
    with pytest.raises(AssertionError, match="SymmetricMemory"):
        all_gather_matmul_tma_persistent(a_out[:128].clone(), b, a_out, c_out, None)
    with pytest.raises(AssertionError):
        all_gather_matmul_tma_persistent(a_shard, b[:, :32].contiguous(), a_out, c_out, None)
    with pytest.raises(AssertionError):
        all_gather_matmul_tma_persistent(a_shard, b, a_out, c_out, {"BLOCK_SIZE_M": 128, "GROUP_SIZE_M": 4})


def test_full_size_config5(cuda):
    """M=16384 N=3584 K=8192 (8 shards of [2048, 8192]), fused, rank 0.  The full
    product costs ~1 TFLOP on the CPU, so the oracle is evaluated on 96 rows that
    touch every shard and every 256-row tile boundary class, over all columns;
    the remaining rows are covered by a linearity check against an independent
    fp32 matvec: C @ 1 == A @ (B^T @ 1)."""
    from symm_mem_recipes import all_gather_matmul_tma_persistent
    M, N, K, ws = 16384, 3584, 8192, 8
    a_shard, h, shards, b, b_bits, a_out, c_out = _setup(M, N, K, ws, 0, cuda)
    all_gather_matmul_tma_persistent(a_shard, b, a_out, c_out, None)
    h.check_status()
    rows = sorted({s * 2048 + o for s in range(ws) for o in (0, 1, 255, 256, 1023, 1024, 1279, 1500, 1792, 2046, 2047, 31)})
    a_all = np.concatenate(shards)
    want = O.ag_matmul_ref([a_all[rows]], b_bits)
    _check(_t_bits(c_out[rows]), want)
    assert np.array_equal(_t_bits(a_out[rows]), a_all[rows])
    a_gpu = torch.cat([h.get_buffer(r, (M // ws, K), torch.bfloat16) for r in range(ws)]).float()
    rowsum = a_gpu @ b.float().sum(dim=0)
    got = c_out.float().sum(dim=1)
    # every entry carries at most half a bf16 ulp of rounding; over N entries the
    # errors add like a random walk: allow 8 standard deviations
    c_rms = float(c_out.float().pow(2).mean().sqrt())
    tol = 8 * (N ** 0.5) * 2.0 ** -9 * c_rms + 1e-3
    assert torch.all((got - rowsum).abs() <= tol), float((got - rowsum).abs().max())


@pytest.mark.parametrize("M,N,K", [(16384, 1792, 4096), (8192, 3584, 8192), (32768, 1792, 2048)])
def test_fused_launch_at_full_size_gathers_every_row(cuda, M, N, K):
    """The fused launch at sizes where its workgroups copy between two tiles with every register
    taken: the gathered operand equals the shards and the product equals that of the
    copy-then-multiply form bit for bit.  (In the e4m3fn kernel a register the compiler reloaded
    right behind one of the copy's assembly stores once changed what was stored, at the first of
    these shapes only.)"""
    from symm_mem_recipes import all_gather_matmul_tma_persistent
    ws = 8
    a_shard, h, shards, b, b_bits, a_out, c_out = _setup(M, N, K, ws, 3, cuda)
    want_a = np.concatenate(shards)
    for _ in range(3):
        a_out.fill_(float("nan"))
        all_gather_matmul_tma_persistent(a_shard, b, a_out, c_out, None, fused=True)
        h.check_status()
        assert np.array_equal(_t_bits(a_out), want_a)
        fused_bits = _t_bits(c_out)
        c_out.fill_(float("nan"))
        a_out.fill_(float("nan"))
        all_gather_matmul_tma_persistent(a_shard, b, a_out, c_out, None, fused=False)
        h.check_status()
        assert np.array_equal(_t_bits(a_out), want_a)
        assert np.array_equal(fused_bits, _t_bits(c_out))


def test_golden_vectors(cuda):
    """tests/golden/ag_matmul.npz: 4 shards of [128, 64], B [72, 64]."""
    import os
    from symm_mem_recipes import EmulatedSymmetricMemory as SM, all_gather_matmul_tma_persistent
    g = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "ag_matmul.npz"))
    ws, rows, K = g["shards"].shape
    N = g["b_nk"].shape[0]
    for rank in range(ws):
        a_shard = SM.empty_strided_p2p((rows, K), (K, 1), torch.bfloat16, cuda, world_size=ws, rank=rank)
        h = SM.rendezvous(a_shard)
        for r in range(ws):
            h.get_buffer(r, (rows, K), torch.bfloat16).copy_(_bits_t(g["shards"][r]))
        a_out = torch.zeros(ws * rows, K, dtype=torch.bfloat16, device=cuda)
        c_out = torch.full((ws * rows, N), float("nan"), dtype=torch.bfloat16, device=cuda)
        all_gather_matmul_tma_persistent(a_shard, _bits_t(g["b_nk"]).to(cuda), a_out, c_out, None)
        h.check_status()
        _check(_t_bits(c_out), g["c"])
