"""GPU parity of the split-K GEMV + flag-combined reduce against the CPU oracle.
No reference code or vectors exist for this path (parity unpinned against the
reference); the oracle is the closed form, pinned on the CPU against x @ W and
exact rational arithmetic.  Tolerance: the fp32 partials may differ from the
oracle's correctly rounded ones by accumulated fp32 rounding (|err| <= 1e-5 of
the sum of |terms|); the bf16 output must be within 1 bf16 ulp and within 1e-2
relative."""
import numpy as np
import pytest
import torch

from oracle import oracle as O

pytestmark = pytest.mark.gpu


def _bits_t(bits):
    return torch.from_numpy(bits.view(np.int16).copy()).view(torch.bfloat16)


def _t_bits(t):
    return t.contiguous().view(torch.int16).cpu().numpy().view(np.uint16)


def _bf16_ulp(v):
    """Spacing of bf16 at |v| (normal range)."""
    return 2.0 ** (np.floor(np.log2(np.maximum(np.abs(v), 2.0 ** -126))) - 7)


def _within_one_ulp(got, ref, term_sum):
    """|got - ref| <= 1 bf16 ulp (of the larger binade of the two, for results that
    straddle a power of two) + the fp32 accumulation slack 1e-5 * sum |x||w|, which
    matters only where the terms cancel to almost nothing."""
    tol = np.maximum(_bf16_ulp(got), _bf16_ulp(ref)) + 1e-5 * term_sum
    return np.all(np.abs(got - ref) <= tol)


@pytest.fixture(params=[(0, 0, 1), (0, 0, 0), (0, 2, 1), (64, 0, 1), (64, 3, 1)],
                ids=["default", "vector-only", "2sub", "wide", "wide-3sub"])
def launch_shape(request, lib):
    """Launch shapes: the default (batches above 2 on the matrix cores where the K rows of a
    workgroup are whole 32-row tiles), every batch on the vector ALUs, K sub-shards, and the
    64-thread row segments."""
    tpr, sub, matrix = request.param
    assert lib.smr_set_gemv_launch(tpr, sub) == 0
    assert lib.smr_set_gemv_matrix_cores(matrix) == 0
    yield request.param
    lib.smr_set_gemv_launch(0, 0)
    lib.smr_set_gemv_matrix_cores(1)


@pytest.mark.parametrize("batch,K,N,ws", [(1, 512, 128, 8), (4, 1024, 256, 8), (8, 2048, 1000, 8),
                                          (3, 768, 136, 4), (8, 8192, 384, 8), (5, 16384, 128, 8)])
def test_gemv_parity(cuda, launch_shape, batch, K, N, ws):
    from symm_mem_recipes import gemv_all_reduce, GemvWorkspace
    x_bits = O.seeded_normal_bf16_bits(batch * K, seed=0).reshape(batch, K)
    w_bits = O.seeded_normal_bf16_bits(K * N, seed=1, std=0.02).reshape(K, N)
    x = _bits_t(x_bits).to(cuda)
    w = _bits_t(w_bits).to(cuda)
    wsp = GemvWorkspace(batch, N, ws, cuda, K)
    senders = wsp.senders
    assert senders % ws == 0
    sub = senders // ws                     # the kernel may cut a rank's K shard into sub-shards
    want, want_partials = O.gemv_allreduce_ref(x_bits, w_bits, ws, return_partials=True)
    for _ in range(2):                      # second call: flags must have returned to zero
        out = gemv_all_reduce(x, w, ws, wsp)
        wsp.check_status()
        assert int(wsp.flags.abs().sum().item()) == 0
        got_p = wsp.partials.cpu().numpy()[:senders]
        per_rank = got_p.reshape(ws, sub, batch, N).astype(np.float64).sum(axis=1)
        xf = np.abs(O.bf16_bits_to_f32(x_bits)).astype(np.float64)
        wf = np.abs(O.bf16_bits_to_f32(w_bits)).astype(np.float64)
        ks = K // ws
        for r in range(ws):
            bound = 1e-5 * (xf[:, r * ks:(r + 1) * ks] @ wf[r * ks:(r + 1) * ks]) + 1e-30
            assert np.all(np.abs(per_rank[r] - want_partials[r]) <= bound)
        got = O.bf16_bits_to_f32(_t_bits(out)).astype(np.float64)
        ref = O.bf16_bits_to_f32(want).astype(np.float64)
        assert _within_one_ulp(got, ref, xf @ wf)
        rms = np.sqrt(np.mean(ref ** 2))
        assert np.all(np.abs(got - ref) <= 1e-2 * np.abs(ref) + 1e-2 * rms)
        # the combine itself is exact: fp32 sum of the kernel's own partials in sender
        # order (rank-major)
        acc = np.zeros_like(got_p[0])
        for r in range(senders):
            acc = (acc + got_p[r]).astype(np.float32)
        assert np.array_equal(_t_bits(out), O.f32_to_bf16_bits(acc))


def test_gemv_config4_full_size(cuda):
    """x [8, 8192], W [8192, 8192], 8 K-shards of 1024 rows."""
    from symm_mem_recipes import gemv_all_reduce, GemvWorkspace
    K = N = 8192
    x_bits = O.seeded_normal_bf16_bits(8 * K, seed=0).reshape(8, K)
    w_bits = O.seeded_normal_bf16_bits(K * N, seed=1, std=0.02).reshape(K, N)
    x, w = _bits_t(x_bits).to(cuda), _bits_t(w_bits).to(cuda)
    want = O.gemv_allreduce_ref(x_bits, w_bits, 8)
    terms = np.abs(O.bf16_bits_to_f32(x_bits)).astype(np.float64) @ np.abs(O.bf16_bits_to_f32(w_bits)).astype(np.float64)
    for batch in (1, 4, 8):
        wsp = GemvWorkspace(batch, N, 8, cuda, K)
        out = gemv_all_reduce(x[:batch].contiguous(), w, 8, wsp)
        wsp.check_status()
        got = O.bf16_bits_to_f32(_t_bits(out)).astype(np.float64)
        ref = O.bf16_bits_to_f32(want[:batch]).astype(np.float64)
        assert _within_one_ulp(got, ref, terms[:batch])
        rms = np.sqrt(np.mean(ref ** 2))
        assert np.all(np.abs(got - ref) <= 1e-2 * np.abs(ref) + 1e-2 * rms)


def test_gemv_validation(cuda):
    from symm_mem_recipes import gemv_all_reduce
    x = torch.zeros(9, 64, dtype=torch.bfloat16, device=cuda)
    w = torch.zeros(64, 128, dtype=torch.bfloat16, device=cuda)
    with pytest.raises(AssertionError, match="batch"):
        gemv_all_reduce(x, w)
    with pytest.raises(AssertionError, match="split evenly"):
        gemv_all_reduce(x[:2, :60].contiguous(), w[:60].contiguous())
    with pytest.raises(AssertionError):
        gemv_all_reduce(x[:2].contiguous(), w[:, :100].contiguous())       # N % 8


def test_golden_vectors(cuda):
    """tests/golden/gemv.npz: x [4, 256], W [256, 128], 8 K-shards."""
    import os
    from symm_mem_recipes import gemv_all_reduce
    g = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "gemv.npz"))
    out = gemv_all_reduce(_bits_t(g["x"]).to(cuda), _bits_t(g["w"]).to(cuda), 8)
    torch.cuda.synchronize()
    got = O.bf16_bits_to_f32(_t_bits(out)).astype(np.float64)
    ref = O.bf16_bits_to_f32(g["out"]).astype(np.float64)
    terms = np.abs(O.bf16_bits_to_f32(g["x"])).astype(np.float64) @ np.abs(O.bf16_bits_to_f32(g["w"])).astype(np.float64)
    assert _within_one_ulp(got, ref, terms)


def test_gemv_replays_from_a_graph(cuda):
    """Three launches on one workspace captured into a HIP graph (kernel nodes only):
    every replay, with eager work and synchronisations in between, gives the eager bits,
    and the flags are back to zero for the next."""
    from symm_mem_recipes import gemv_all_reduce, GemvWorkspace
    batch, K, N, ws = 4, 2048, 1024, 8
    g = torch.Generator(device=cuda)
    g.manual_seed(5)
    x = torch.empty(batch, K, device=cuda).normal_(0, 1, generator=g).to(torch.bfloat16)
    w = torch.empty(K, N, device=cuda).normal_(0, 0.02, generator=g).to(torch.bfloat16)
    work = GemvWorkspace(batch, N, ws, cuda, K)
    eager = gemv_all_reduce(x, w, ws, work).clone()
    work.check_status()
    outs = [torch.empty(batch, N, dtype=torch.bfloat16, device=cuda) for _ in range(3)]
    side = torch.cuda.Stream(cuda)
    side.wait_stream(torch.cuda.current_stream(cuda))
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            for o in outs:
                gemv_all_reduce(x, w, ws, work, out=o)
    torch.cuda.current_stream(cuda).wait_stream(side)
    for replay in range(4):
        for o in outs:
            o.zero_()
        noise = torch.randn(1 << 18, device=cuda).sum()
        torch.cuda.synchronize()
        graph.replay()
        work.check_status()
        assert int(work.flags.abs().sum()) == 0
        for o in outs:
            assert torch.equal(o.view(torch.int16), eager.view(torch.int16)), replay
        del noise
    del graph
