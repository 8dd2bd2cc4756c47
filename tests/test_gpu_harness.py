"""The timing harness and the modules' self-checks, as the reference runs them
(symm_mem_recipes/utils.py:10-134; the __main__ blocks of its three kernel modules)."""
import importlib

import pytest
import torch

pytestmark = pytest.mark.gpu


def test_benchmark_with_event_times_a_known_delay(cuda):
    from symm_mem_recipes import utils
    cycles = int(0.5 * utils._cycles_per_ms())                     # a device-side spin of about 500 us
    for flush in (False, True):
        us = utils.benchmark_with_event(lambda: torch.cuda._sleep(cycles), warmup_iters=3,
                                        benchmark_iters=5, flush_l2=flush)
        assert 350 < us < 900, us
    from symm_mem_recipes import set_rank
    set_rank(1)                                                    # a rank that does not report
    try:
        assert utils.benchmark_with_event(lambda: None, warmup_iters=1, benchmark_iters=2) == 0
    finally:
        set_rank(0)


def test_benchmark_with_profiler_finds_the_reduce_kernel(cuda):
    from symm_mem_recipes import EmulatedSymmetricMemory as SM, one_shot_all_reduce, utils
    t = SM.empty_strided_p2p((8192,), (1,), torch.bfloat16, cuda, world_size=8)
    h = SM.rendezvous(t)
    for r in range(8):
        h.get_buffer(r, (8192,), torch.bfloat16).fill_(1)
    us = utils.benchmark_with_profiler(lambda: one_shot_all_reduce(t), r".*one_shot_all_reduce_kernel",
                                       warmup_iters=5, benchmark_iters=20)
    assert 1 < us < 100, us
    assert utils.benchmark_with_profiler(lambda: one_shot_all_reduce(t), r"no_such_kernel",
                                         warmup_iters=1, benchmark_iters=2) == 0
    h.check_status()
    SM.release(t)


def test_module_self_checks(cuda, capsys):
    """ones -> world_size with a latency line; the barrier returns and leaves zeros; the
    fused GEMM agrees with gather + library matmul and prints four latencies."""
    importlib.import_module("symm_mem_recipes.one_shot_all_reduce").main()
    assert "Median latency:" in capsys.readouterr().out
    importlib.import_module("symm_mem_recipes.barrier").main()
    assert "tensor([0, 0, 0" in capsys.readouterr().out
    importlib.import_module("symm_mem_recipes.all_gather_matmul").main(
        ["--M", "4096", "--N", "512", "--K", "1024"])
    out = capsys.readouterr().out
    for label in ("library matmul only:", "hip matmul only:", "library gather + matmul:", "hip all_gather_matmul:"):
        assert label in out


def test_trace_of_a_launch(cuda):
    """The kernels' own time stamps: every workgroup's tiles in order, the producer's flags
    behind its start, and the fused launch's first wait no longer than the whole launch."""
    from symm_mem_recipes import trace
    for mode in ("ungated", "fused", "streams", "sequential"):
        r = trace.trace_launch(16384, 2048, 256, mode, warm=2)
        assert r["end_us"] > 0 and r["steps"], mode
        assert sum(s["workgroups"] for s in r["steps"]) == (16384 // 256) * (2048 // 256), mode
        for s in r["steps"]:
            assert s["k_loop_us"] > 0 and s["wait_us"] >= 0 and s["last_stored_us"] <= r["end_us"]
        if mode in ("fused", "streams"):
            assert r["producer_start_us"] is not None and len(r["flags_us"]) >= 6
            assert all(v > r["producer_start_us"] for v in r["flags_us"].values())


def test_mfma_only_probe(cuda):
    """The measurement aid behind the bench's "mfma_only" figure: it runs, every workgroup
    reports its two clocks, and back-to-back MFMAs issue at 16 cycles apiece (a little more
    with the loop's branch), which is what the figure's FLOP count assumes."""
    from symm_mem_recipes import _lib
    lib = _lib.load_probe()
    wgs, iters = 16, 2000
    vals = torch.empty(4096, dtype=torch.bfloat16, device=cuda).normal_(0, 0.02)
    ticks = torch.zeros(2 * wgs, dtype=torch.int64, device=cuda)
    sink = torch.zeros(256 * wgs, dtype=torch.float32, device=cuda)
    st = torch.cuda.current_stream(cuda).cuda_stream
    assert lib.smr_probe_mfma_only(vals.data_ptr(), vals.numel(), wgs, iters, ticks.data_ptr(), sink.data_ptr(), st) == 0
    torch.cuda.synchronize()
    t = ticks.view(wgs, 2).cpu()
    assert bool((t > 0).all())
    per_mfma = t[:, 1].double() / (64.0 * iters)
    assert 15.9 <= per_mfma.min().item() and per_mfma.max().item() <= 20.0, per_mfma.tolist()
    assert torch.isfinite(sink).all()
    assert lib.smr_probe_mfma_only(None, 1, 1, 1, ticks.data_ptr(), sink.data_ptr(), st) == -1
    assert lib.smr_probe_mfma_only(vals.data_ptr(), 0, 1, 1, ticks.data_ptr(), sink.data_ptr(), st) == -1
