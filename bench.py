#!/usr/bin/env python3
"""Benchmark of the symmetric-memory hot path on one MI355X.

A "step" is one one-shot all-reduce over 8 emulated peer buffers of bf16 resident
in HBM (single output: one GPU's real share of the job).  Prints ONE JSON line:
the reduce throughput in GB/s with its HBM roofline, the CPU baseline (the numpy
oracle timed on the host), and under "extra" the other kernels of the path
(flag-gated all-gather matmul against the bf16 MFMA roofline, split-K GEMV,
barrier / signal-pad rounds, smaller reduce sizes with rotating buffer sets).

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--size-mib S] [--no-extra]
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for _p in (ROOT, os.path.join(ROOT, "symm-mem-recipes_amd")):
    if _p not in sys.path:
        sys.path.insert(0, _p)

HBM_PEAK_GBS = 8000.0          # MI355X HBM3E, published
MFMA_BF16_PEAK_TFLOPS = 2500.0  # MI355X dense bf16, published
MFMA_FP8_PEAK_TFLOPS = 5000.0   # MI355X dense fp8, published
WS = 8


def _counters():
    """Hardware-counter figures that a timing run cannot take itself, from the file written next
    to the rocprofv3 summaries they come from (profiles/counters.json; every entry names its
    summary).  reduce_traffic_bytes: memory bytes per launch of the reduce kernel (FETCH_SIZE /
    WRITE_SIZE, each scaled by what the counter reads for this script's 512 MiB calibration
    copy), keyed by MiB per buffer.  gemm / gemm_fp8: per launch at M=16384 N=3584 K=8192,
    "traffic" = bytes between the XCDs' L2s and the fabric (the 256 MiB last-level cache serves
    part of it, so it is not HBM traffic), "mfma_busy" = SQ_VALU_MFMA_BUSY_CYCLES per SIMD over
    the launch's elapsed shader cycles.  A missing file or entry gives null in the output."""
    try:
        with open(os.path.join(ROOT, "profiles", "counters.json")) as f:
            return json.load(f)
    except (OSError, ValueError):
        return {}


def _median(xs):
    xs = sorted(xs)
    return xs[len(xs) // 2]


def _time_events(fn, iters, warm, pre=None):
    """Median device time of fn() in microseconds, one event pair per call on the
    launch stream; `pre` (for example a cache flush) runs before each timed call."""
    import torch
    for _ in range(warm):
        fn()
    torch.cuda.synchronize()
    ts = []
    for _ in range(iters):
        if pre is not None:
            pre()
        a = torch.cuda.Event(enable_timing=True)
        b = torch.cuda.Event(enable_timing=True)
        a.record()
        fn()
        b.record()
        torch.cuda.synchronize()
        ts.append(a.elapsed_time(b) * 1e3)
    return _median(ts)


def _time_batched(fn, calls, warm, batches=3):
    """Device time per call in microseconds over `calls` back-to-back launches between one event
    pair - for kernels of a few tens of microseconds, where a synchronise after every call would
    time the launch path instead - as the median of `batches` such batches."""
    import torch
    for _ in range(warm):
        fn()
    torch.cuda.synchronize()
    per_call = []
    for _ in range(batches):
        a = torch.cuda.Event(enable_timing=True)
        b = torch.cuda.Event(enable_timing=True)
        a.record()
        for _ in range(calls):
            fn()
        b.record()
        torch.cuda.synchronize()
        per_call.append(a.elapsed_time(b) * 1e3 / calls)
    return _median(per_call)


def bench_reduce(size_mib, steps, warmup, dev):
    import torch
    from symm_mem_recipes import EmulatedSymmetricMemory as SM, one_shot_all_reduce
    nbytes = size_mib << 20
    numel = nbytes // 2
    t = SM.empty_strided_p2p((numel,), (1,), torch.bfloat16, dev, world_size=WS, rank=0)
    h = SM.rendezvous(t)
    g = torch.Generator(device=dev)
    for r in range(WS):
        g.manual_seed(r)
        h.get_buffer(r, (numel,), torch.bfloat16).normal_(generator=g)
    # The headline is the reference's call as the drop-in ships it: the blockwise barrier, then
    # the reduce (triton_one_shot_all_reduce.py:70-93).
    out = None
    for _ in range(warmup):
        out = one_shot_all_reduce(t)
    torch.cuda.synchronize()
    e0 = torch.cuda.Event(enable_timing=True)
    e1 = torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    e0.record()
    for _ in range(steps):
        out = one_shot_all_reduce(t)
    e1.record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    h.check_status()
    dev_us = e0.elapsed_time(e1) * 1e3 / steps
    alg_bytes = (WS + 1) * nbytes
    # the same reduce without the handshake (peers' data already stream-ordered), timed the way
    # the headline is (back-to-back launches between one event pair), and the write-back-to-all variant
    us_no_barrier = _time_batched(lambda: one_shot_all_reduce(t, barrier=False), max(steps // 2, 10), 3)
    us_write_all = _time_events(lambda: one_shot_all_reduce(t, barrier=False, write_all=True), 20, 3)
    # two-shot: every emulated rank reduces its eighth and writes it to all peers, two handshakes
    for r in range(WS):
        g.manual_seed(r)
        h.get_buffer(r, (numel,), torch.bfloat16).normal_(generator=g)
    us_two_shot = _time_events(lambda: one_shot_all_reduce(t, all_ranks=True, write_all=True), 12, 3)
    h.check_status()
    SM.release()
    del out
    return dict(wall_s=wall, dev_us=dev_us, alg_bytes=alg_bytes, us_no_barrier=us_no_barrier,
                us_write_all=us_write_all, write_all_bytes=2 * WS * nbytes, us_two_shot=us_two_shot)


def bench_reduce_rotating(size_kib, dev, dtype_name="bf16", write_all=False, accumulate="fp32", barrier=False):
    """Messages below 64 MiB fit the 256 MB last-level cache; rotate over enough buffer
    sets (1 GiB in total, at most 64 sets) that every call reads from HBM."""
    import torch
    from symm_mem_recipes import EmulatedSymmetricMemory as SM, one_shot_all_reduce
    dtype = torch.bfloat16 if dtype_name == "bf16" else torch.float32
    nbytes = size_kib << 10
    numel = nbytes // (2 if dtype == torch.bfloat16 else 4)
    nsets = min(64, max(2, -(-(1 << 30) // (WS * nbytes))))
    sets = []
    for _ in range(nsets):
        t = SM.empty_strided_p2p((numel,), (1,), dtype, dev, world_size=WS, rank=0)
        h = SM.rendezvous(t)
        for r in range(WS):
            h.get_buffer(r, (numel,), dtype).normal_()
        sets.append(t)
    idx = [0]

    def call():
        one_shot_all_reduce(sets[idx[0] % nsets], barrier=barrier, write_all=write_all, accumulate=accumulate)
        idx[0] += 1
    us = _time_batched(call, max(10 * nsets, 200), nsets)
    alg = (2 * WS if write_all else WS + 1) * nbytes
    res = dict(size_kib=size_kib, dtype=dtype_name, mode="write_all" if write_all else "single_output",
               accumulate=accumulate, us=us, gbs=alg / us / 1e3, frac=alg / us / 1e3 / HBM_PEAK_GBS,
               buffer_sets=nsets)
    if barrier:
        res["mode"] += ", behind the blockwise barrier"
    if nbytes <= (4 << 20) and not write_all and not barrier:
        # Below a few MiB the eager figure is the host's launch rate, not the kernel:
        # replay one pass over the buffer sets from a HIP graph (kernel nodes only) and
        # check every replay against the eager result.
        ref = one_shot_all_reduce(sets[0], barrier=False, accumulate=accumulate).clone()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            outs = [one_shot_all_reduce(t, barrier=False, accumulate=accumulate) for t in sets]
        reps = max(4, 400 // nsets)
        for _ in range(2):
            graph.replay()
            torch.cuda.synchronize()
            assert torch.equal(outs[0], ref), "graph replay differs from the eager result"
        a = torch.cuda.Event(enable_timing=True)
        b = torch.cuda.Event(enable_timing=True)
        a.record()
        for _ in range(reps):
            graph.replay()
        b.record()
        torch.cuda.synchronize()
        assert torch.equal(outs[0], ref), "graph replay differs from the eager result"
        res["us_graph_replay"] = a.elapsed_time(b) * 1e3 / (reps * nsets)
        del graph, outs
    SM.release()
    return res


def _time_interleaved(fns, iters, warm, pre=None):
    """Median device time in microseconds of each fn in `fns`, one call of each per round in
    an order drawn afresh for every round (seeded): variants measured one block after another
    see different clocks, because the part's power management reacts to the last milliseconds
    of load, and in a fixed order every variant would always run behind the same other one."""
    import random
    import torch
    for _ in range(warm):
        for fn in fns:
            fn()
    torch.cuda.synchronize()
    ts = [[] for _ in fns]
    rng = random.Random(0)
    for _ in range(iters):
        order = list(enumerate(fns))
        rng.shuffle(order)
        for k, fn in order:
            if pre is not None:
                pre()
            a = torch.cuda.Event(enable_timing=True)
            b = torch.cuda.Event(enable_timing=True)
            a.record()
            fn()
            b.record()
            torch.cuda.synchronize()
            ts[k].append(a.elapsed_time(b) * 1e3)
    return [_median(t) for t in ts]


def bench_mfma_only(dev):
    """What the matrix cores sustain with every compute unit issuing bf16 MFMAs back to back on
    N(0, 0.02) operands and nothing else (smr_probe_mfma_only): the part's power management
    sets the clock, so this - not the published peak, which assumes the top clock - is what
    the GEMM's MFMA share can be compared with."""
    import torch
    from symm_mem_recipes import _lib
    lib = _lib.load_probe()
    cus = torch.cuda.get_device_properties(dev).multi_processor_count
    vals = torch.empty(1 << 16, dtype=torch.bfloat16, device=dev).normal_(0, 0.02)
    ticks = torch.zeros(2 * cus, dtype=torch.int64, device=dev)
    sink = torch.zeros(256 * cus, dtype=torch.float32, device=dev)
    iters = 20000                                  # about 10 ms per launch: time for the clock to settle
    st = torch.cuda.current_stream(dev).cuda_stream
    for _ in range(4):
        rc = lib.smr_probe_mfma_only(vals.data_ptr(), vals.numel(), cus, iters, ticks.data_ptr(), sink.data_ptr(), st)
        assert rc == 0
    torch.cuda.synchronize()
    t = ticks.view(cus, 2).double()
    us = (t[:, 0] / 100.0).mean().item()
    flops = cus * 4.0 * 64 * iters * 16384
    return {"tflops": flops / us / 1e6, "shader_clock_mhz": (t[:, 1].mean() / us).item(),
            "cycles_per_mfma": (t[:, 1].mean() / (64.0 * iters)).item(), "workgroups": cus}


def bench_ag_matmul(dev, gated=True, two_streams=True):
    import torch
    counters = _counters().get("gemm", {})
    from symm_mem_recipes import EmulatedSymmetricMemory as SM, _lib, all_gather_matmul_tma_persistent
    lib = _lib.load()
    M, N, K = 16384, 3584, 8192
    a_shard = SM.empty_strided_p2p((M // WS, K), (K, 1), torch.bfloat16, dev, world_size=WS, rank=0)
    h = SM.rendezvous(a_shard)
    g = torch.Generator(device=dev)
    for r in range(WS):
        g.manual_seed(r)
        h.get_buffer(r, (M // WS, K), torch.bfloat16).normal_(0, 0.02, generator=g)
    g.manual_seed(100)
    b = torch.empty(N, K, dtype=torch.bfloat16, device=dev).normal_(0, 0.02, generator=g)
    a_out = torch.cat([h.get_buffer(r, (M // WS, K), torch.bfloat16) for r in range(WS)]).contiguous()
    c = torch.empty(M, N, dtype=torch.bfloat16, device=dev)
    flush = torch.empty(1 << 28, dtype=torch.int32, device=dev)      # 1 GiB > last-level cache
    flops = 2.0 * M * N * K
    gated_grid = lib.smr_ag_matmul_grid(M, N, K, WS, M // WS, 1)

    def ungated_on_the_gated_grid():
        # the ungated launch held to the workgroups (and so the tiles) of the gated one: what the
        # flags themselves cost is the gated launch against THIS; the whole-GPU launch below is
        # also ahead by the compute units that the copy occupies on one GPU
        lib.smr_set_ag_matmul_grid_limit(gated_grid)
        try:
            all_gather_matmul_tma_persistent(a_shard, b, a_out, c, None, mm_only=True)
        finally:
            lib.smr_set_ag_matmul_grid_limit(0)

    fns = [lambda: all_gather_matmul_tma_persistent(a_shard, b, a_out, c, None, mm_only=True),
           lambda: torch.matmul(a_out, b.T, out=c), ungated_on_the_gated_grid]
    if gated:
        fns.append(lambda: all_gather_matmul_tma_persistent(a_shard, b, a_out, c, None))
    streams_error = None
    if gated and two_streams:
        # The two-stream form needs its two kernels side by side; a profiler that serialises
        # kernels makes the GEMM's bounded waits expire.  One checked call decides whether it is timed.
        try:
            all_gather_matmul_tma_persistent(a_shard, b, a_out, c, None, fused="streams", check=True)
            fns.append(lambda: all_gather_matmul_tma_persistent(a_shard, b, a_out, c, None, fused="streams"))
        except _lib.SmrError as exc:
            streams_error = repr(exc)[:200]
    us = _time_interleaved(fns, 25, 10, pre=flush.zero_)
    us_ungated, us_lib, us_same_grid = us[0], us[1], us[2]
    us_gated = us[3] if gated else float("nan")
    us_streams = us[4] if len(us) > 4 else float("nan")
    h.check_status()
    SM.release()
    return dict(workload="all-gather matmul M=16384 N=3584 K=8192 bf16, 8 shards of [2048, 8192], rank 0",
                flops=flops, us_gated=us_gated, us_ungated=us_ungated,
                us_ungated_on_the_gated_grid=us_same_grid, gated_grid=gated_grid,
                us_two_streams=us_streams, tflops_two_streams=flops / us_streams / 1e6,
                two_streams_error=streams_error,
                tflops_gated=flops / us_gated / 1e6, tflops_ungated=flops / us_ungated / 1e6,
                frac_ungated=flops / us_ungated / 1e6 / MFMA_BF16_PEAK_TFLOPS,
                gating_overhead=us_gated / us_same_grid - 1.0,
                gating_overhead_note="fused launch against the ungated launch on the same grid and tiles (the cost "
                                     "of the flags and of the copy's traffic); against the ungated launch that "
                                     "also has the copy's compute units: overhead_vs_whole_gpu",
                overhead_vs_whole_gpu=us_gated / us_ungated - 1.0,
                roofline={"bound": "mfma", "achieved": flops / us_gated / 1e6, "peak": MFMA_BF16_PEAK_TFLOPS,
                          "unit": "TFLOP/s", "frac": flops / us_gated / 1e6 / MFMA_BF16_PEAK_TFLOPS,
                          "traffic": counters.get("fused", {}).get("traffic"),
                          "traffic_kind": "L2 <-> fabric bytes per launch (last-level cache or HBM behind it)",
                          "mfma_busy": counters.get("fused", {}).get("mfma_busy")},
                counters_ungated=counters.get("ungated"),
                counters_ungated_on_the_gated_grid=counters.get("ungated_on_the_gated_grid"),
                counters_hipblaslt=counters.get("hipblaslt"),
                counters_source=counters.get("source"),
                torch_matmul_us=us_lib, torch_matmul_tflops=flops / us_lib / 1e6)


def bench_ag_matmul_fp8(dev, gated=True):
    """The same problem with e4m3fn operands and result (the reference's FP8_OUTPUT switch)."""
    import torch
    from symm_mem_recipes import EmulatedSymmetricMemory as SM, all_gather_matmul_tma_persistent
    M, N, K = 16384, 3584, 8192
    f8 = torch.float8_e4m3fn
    a_shard = SM.empty_strided_p2p((M // WS, K), (K, 1), f8, dev, world_size=WS, rank=0)
    h = SM.rendezvous(a_shard)
    g = torch.Generator(device=dev)
    for r in range(WS):
        g.manual_seed(r)
        h.get_buffer(r, (M // WS, K), f8).copy_(
            torch.empty(M // WS, K, device=dev).normal_(0, 0.05, generator=g).to(f8))
    g.manual_seed(100)
    b = torch.empty(N, K, device=dev).normal_(0, 0.05, generator=g).to(f8)
    a_out = torch.cat([h.get_buffer(r, (M // WS, K), f8) for r in range(WS)]).contiguous()
    c = torch.empty(M, N, dtype=torch.uint8, device=dev).view(f8)
    flush = torch.empty(1 << 28, dtype=torch.int32, device=dev)
    flops = 2.0 * M * N * K
    fns = [lambda: all_gather_matmul_tma_persistent(a_shard, b, a_out, c, None, mm_only=True)]
    if gated:
        fns.append(lambda: all_gather_matmul_tma_persistent(a_shard, b, a_out, c, None))
    us = _time_interleaved(fns, 25, 10, pre=flush.zero_)
    us_ungated, us_gated = us[0], (us[1] if gated else float("nan"))
    h.check_status()
    res = dict(workload="all-gather matmul M=16384 N=3584 K=8192 e4m3fn in and out, 8 shards of [2048, 8192], rank 0",
               flops=flops, us_gated=us_gated, us_ungated=us_ungated,
               tflops_gated=flops / us_gated / 1e6, tflops_ungated=flops / us_ungated / 1e6,
               gating_overhead=us_gated / us_ungated - 1.0,
               roofline={"bound": "mfma", "achieved": flops / us_gated / 1e6, "peak": MFMA_FP8_PEAK_TFLOPS,
                         "unit": "TFLOP/s", "frac": flops / us_gated / 1e6 / MFMA_FP8_PEAK_TFLOPS,
                         "traffic": _counters().get("gemm_fp8", {}).get("fused", {}).get("traffic")})
    try:                                            # the library's fp8 GEMM of the same operands (bf16 result)
        one = torch.ones((), device=dev)
        us_lib = _time_events(lambda: torch._scaled_mm(a_out, b.T, scale_a=one, scale_b=one,
                                                       out_dtype=torch.bfloat16), 25, 20, pre=flush.zero_)
        res.update(torch_scaled_mm_us=us_lib, torch_scaled_mm_tflops=flops / us_lib / 1e6)
    except Exception as exc:                        # not every torch build has it for this dtype
        res["torch_scaled_mm_error"] = repr(exc)[:200]
    SM.release()
    return res


def bench_gemv(dev):
    import torch
    from symm_mem_recipes import GemvWorkspace, gemv_all_reduce
    K = N = 8192
    g = torch.Generator(device=dev)
    g.manual_seed(1)
    nw = 10                                   # rotate over 1.25 GiB of weights
    ws_ = [torch.empty(K, N, dtype=torch.bfloat16, device=dev).normal_(0, 0.02, generator=g) for _ in range(nw)]
    g.manual_seed(0)
    x = torch.empty(8, K, dtype=torch.bfloat16, device=dev).normal_(generator=g)
    res = []
    for batch in (1, 4, 8):
        xb = x[:batch].contiguous()
        wsp = GemvWorkspace(batch, N, WS, dev, K)
        out = torch.empty(batch, N, dtype=torch.bfloat16, device=dev)
        idx = [0]

        def call():
            gemv_all_reduce(xb, ws_[idx[0] % nw], WS, wsp, out)
            idx[0] += 1
        us = _time_batched(call, 5 * nw, nw)
        wsp.check_status()
        nbytes = K * N * 2 + batch * K * 2 + batch * N * 2
        res.append(dict(batch=batch, us=us, gbs=nbytes / us / 1e3, frac=nbytes / us / 1e3 / HBM_PEAK_GBS))
    return res


def bench_barrier(dev):
    import numpy as np
    import torch
    from symm_mem_recipes import EmulatedSymmetricMemory as SM, _lib, blockwise_barrier
    lib = _lib.load()
    blocks, chunk = 304, 65536
    words = chunk // 4
    t = SM.empty_strided_p2p((2 * blocks * words,), (1,), torch.int32, dev, world_size=WS)
    h = SM.rendezvous(t)
    rounds = 10000
    us_flags = _time_events(lambda: blockwise_barrier(h, blocks, rounds), 3, 1) / rounds
    us_flags_only = _time_events(lambda: blockwise_barrier(h, blocks, rounds, order_memory=False), 3, 1) / rounds
    h.check_status()
    src = (torch.rand(WS, blocks, words * 2, device=dev) * 2 - 1).to(torch.bfloat16).view(torch.int32)
    src = src.reshape(WS, blocks, words).contiguous()
    # wrapping uint32 sum of each block's source words, stored as the same bits in int32
    base = src.to(torch.int64).bitwise_and(0xFFFFFFFF).sum(dim=(0, 2)).bitwise_and(0xFFFFFFFF)
    base = (base - (base >= 2 ** 31).to(torch.int64) * 2 ** 32).to(torch.int32)
    sums = torch.zeros(WS, blocks, dtype=torch.int32, device=dev)
    mism = torch.zeros(1, dtype=torch.int32, device=dev)
    prounds = 10000                     # the configuration's 10,000 rounds, payload included
    stream = torch.cuda.current_stream().cuda_stream

    def payload():
        rc = lib.smr_signal_round(src.data_ptr(), h.buffer_ptrs_dev, h.signal_pad_ptrs_dev, base.data_ptr(),
                                  sums.data_ptr(), mism.data_ptr(), WS, blocks, chunk, prounds,
                                  h.status.data_ptr(), stream)
        assert rc == 0
    us_payload = _time_events(payload, 1, 0) / prounds
    h.check_status()
    assert int(mism.item()) == 0, "signal-round checksum mismatch"
    SM.release()
    # One rank's real share: on eight GPUs each runs its own 304 workgroups; the emulation runs
    # all 8 x 304 on one, and the cache write-back and invalidate of an ordered round are served
    # one after the other per XCD, so their cost grows with the workgroups that ask for them.
    # 304 workgroups of a single rank (each handshakes with itself) pay what one GPU would.
    t1 = SM.empty_strided_p2p((1024,), (1,), torch.int32, dev, world_size=1)
    h1 = SM.rendezvous(t1)
    us_one_rank = _time_events(lambda: blockwise_barrier(h1, blocks, 2000), 3, 1) / 2000
    us_one_rank_flags = _time_events(lambda: blockwise_barrier(h1, blocks, 2000, order_memory=False), 3, 1) / 2000
    h1.check_status()
    SM.release()
    written = WS * blocks * chunk
    return dict(workgroups=WS * blocks, rounds_flags=rounds, us_per_round_flags=us_flags,
                us_per_round_flags_no_cache_maintenance=us_flags_only,
                one_rank_share={"workgroups": blocks, "us_per_round_flags": us_one_rank,
                                "us_per_round_flags_no_cache_maintenance": us_one_rank_flags},
                rounds_payload=prounds, us_per_round_payload=us_payload,
                payload_written_mib=written / 2 ** 20, payload_read_mib=WS * written / 2 ** 20,
                payload_gbs=(written + WS * written) / us_payload / 1e3)


def bench_reference_point(dev):
    """The reference's own benchmark point (triton_one_shot_all_reduce.py:145-162): 8192 bf16
    per rank, filled with ones, the call as the reference makes it (behind the blockwise
    barrier), median device time of the kernel over 200 calls from the profiler."""
    import torch
    from symm_mem_recipes import EmulatedSymmetricMemory as SM, one_shot_all_reduce
    from symm_mem_recipes.utils import benchmark_with_profiler
    t = SM.empty_strided_p2p((8192,), (1,), torch.bfloat16, dev, world_size=WS, rank=0)
    h = SM.rendezvous(t)
    for r in range(WS):
        h.get_buffer(r, (8192,), torch.bfloat16).fill_(1)
    assert one_shot_all_reduce(t).eq(WS).all().item()
    h.check_status()
    us = benchmark_with_profiler(lambda: one_shot_all_reduce(t), r".*one_shot_all_reduce_kernel", benchmark_iters=200)
    SM.release()
    return {"workload": "8192 bf16 per rank behind the blockwise barrier, kernel time from the profiler, 200 calls",
            "median_kernel_us": us}


def calibration_copy(dev):
    """A plain device-to-device copy of known size (512 MiB read + 512 MiB written):
    the yardstick against which hardware byte counters are scaled when this script
    runs under a profiler."""
    import torch
    src = torch.empty(512 << 20, dtype=torch.uint8, device=dev).fill_(1)
    dst = torch.empty_like(src)
    us = _time_events(lambda: dst.copy_(src), 5, 2)
    return {"bytes_read": 512 << 20, "bytes_written": 512 << 20, "us": us,
            "gbs": 2 * (512 << 20) / us / 1e3}


def cpu_baseline(budget_s=10.0):
    """The CPU oracle of the reduce on the reference's CPU-runnable case: 8 buffers of
    1,048,576 bf16, N(0,1) seeded per rank, fp32 accumulation in rank order.  Three timings
    of the same arithmetic: the torch restatement (`acc += buf.float()` per rank, cast) on all
    host threads torch uses and on one, and the numpy oracle on one thread."""
    import torch
    from oracle import oracle as O
    from oracle import torch_reduce as T
    n = 1 << 20
    nbytes = (WS + 1) * n * 2

    def timed(fn, seconds):
        fn()
        reps, t0 = 0, time.perf_counter()
        while True:
            fn()
            reps += 1
            el = time.perf_counter() - t0
            if el >= seconds:
                return reps, el

    tens = [T.seeded_normal(n, r) for r in range(WS)]
    all_threads = torch.get_num_threads()
    reps, el = timed(lambda: T.reduce_ref_torch(tens), budget_s * 0.4)
    out = {"value": nbytes * reps / el / 1e9, "unit": "GB/s", "cores": all_threads, "kind": "port",
           "sample": f"{reps} repetitions of the 8 x 1,048,576 bf16 reduce (torch CPU restatement of the oracle, "
                     f"{all_threads} threads) in {el:.1f} s",
           "host_cpus": os.cpu_count()}
    torch.set_num_threads(1)
    try:
        reps, el = timed(lambda: T.reduce_ref_torch(tens), budget_s * 0.3)
    finally:
        torch.set_num_threads(all_threads)
    out["one_thread"] = {"value": nbytes * reps / el / 1e9, "unit": "GB/s", "cores": 1,
                         "sample": f"{reps} repetitions, torch CPU restatement, 1 thread, {el:.1f} s"}
    bufs = [O.seeded_normal_bf16_bits(n, seed=r) for r in range(WS)]
    reps, el = timed(lambda: O.reduce_ref(bufs, "bf16"), budget_s * 0.3)
    out["numpy_one_thread"] = {"value": nbytes * reps / el / 1e9, "unit": "GB/s", "cores": 1,
                               "sample": f"{reps} repetitions, numpy oracle, 1 thread, {el:.1f} s"}
    # the other two paths, once each on a bounded slice (numpy's BLAS uses the host's threads)
    M, N, K = 256, 3584, 8192
    shard = O.seeded_normal_bf16_bits(M * K, seed=0, std=0.02).reshape(M, K)
    b_nk = O.seeded_normal_bf16_bits(N * K, seed=100, std=0.02).reshape(N, K)
    t0 = time.perf_counter()
    O.ag_matmul_ref([shard], b_nk)
    el = time.perf_counter() - t0
    out["ag_matmul"] = {"value": 2.0 * M * N * K / el / 1e12, "unit": "TFLOP/s",
                        "sample": f"{M} of the 16384 rows of the M=16384 N=3584 K=8192 product, once, {el:.2f} s"}
    x = O.seeded_normal_bf16_bits(8 * 8192, seed=0).reshape(8, 8192)
    w = O.seeded_normal_bf16_bits(8192 * 8192, seed=1, std=0.02).reshape(8192, 8192)
    t0 = time.perf_counter()
    O.gemv_allreduce_ref(x, w, WS)
    el = time.perf_counter() - t0
    out["gemv_allreduce"] = {"value": (8192 * 8192 * 2 + 2 * 8 * 8192 * 2) / el / 1e9, "unit": "GB/s",
                             "sample": f"batch 8, K = N = 8192, 8 K-shards, once, {el:.2f} s"}
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--size-mib", type=int, default=64)
    ap.add_argument("--no-extra", action="store_true")
    ap.add_argument("--cpu-seconds", type=float, default=10.0)
    ap.add_argument("--gemm-only", action="store_true",
                    help="only the GEMM of the all-gather matmul (ungated, the library's matmul of the same "
                         "operands, and the fused launch): the run to collect hardware counters on")
    ap.add_argument("--fp8", action="store_true", help="with --gemm-only: the e4m3fn GEMM instead of the bf16 one")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on exactly one GPU (the 8 ranks are emulated in one "
              "MI355X's HBM); --gpus must be 1", file=sys.stderr)
        sys.exit(2)

    import torch
    from symm_mem_recipes import _lib
    _lib.load()                                   # fails loudly when the HIP library is missing
    assert torch.cuda.is_available(), "bench.py needs a GPU"
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)

    if args.gemm_only:
        # (kernels only, one stream: this is the run hardware counters are collected on)
        print(json.dumps(bench_ag_matmul_fp8(dev) if args.fp8 else bench_ag_matmul(dev, two_streams=False)))
        return

    r = bench_reduce(args.size_mib, args.steps, args.warmup, dev)
    value = r["alg_bytes"] * args.steps / r["wall_s"] / 1e9
    achieved = r["alg_bytes"] / r["dev_us"] / 1e3
    line = {
        "metric": "one-shot all-reduce GB/s, 8 x bf16 peer buffers (algorithmic bytes 9*S per call), "
                  "behind the blockwise barrier as the reference calls it",
        "value": value,
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": r["wall_s"] * 1e3 / args.steps,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": f"one-shot all-reduce, 8 emulated peer buffers of {args.size_mib} MiB bf16 "
                               "N(0,1) seeded per rank, resident in HBM, blockwise barrier then single output, "
                               "fp32 accumulation in rank order", "world_size": WS,
                    "bytes_per_buffer": args.size_mib << 20},
        "roofline": {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": achieved / HBM_PEAK_GBS,
                     "traffic": _counters().get("reduce_traffic_bytes", {}).get(str(args.size_mib))},
    }
    extra = {
        "reduce_kernel_us": r["dev_us"],
        "reduce_without_barrier_us": r["us_no_barrier"],
        "reduce_without_barrier_frac": r["alg_bytes"] / r["us_no_barrier"] / 1e3 / HBM_PEAK_GBS,
        "reduce_write_all_us": r["us_write_all"],
        "reduce_write_all_gbs": r["write_all_bytes"] / r["us_write_all"] / 1e3,
        "reduce_two_shot_us": r["us_two_shot"],
        "reduce_two_shot_gbs": r["write_all_bytes"] / r["us_two_shot"] / 1e3,
    }
    extra["calibration_copy"] = calibration_copy(dev)
    if not args.no_extra:
        # The size sweep on rotating buffer sets; 2 and 8 MiB are the points the targets name.
        # The cases that stream from HBM (8 MiB per buffer and up) run first, each group largest
        # first: their buffer sets (1 GiB per case) are then carved from the segments the first
        # cases left with torch's caching allocator, as a process that allocates its symmetric
        # buffers at start-up would have them, instead of from whatever the driver finds next to
        # gigabytes of smaller cached blocks (8 MiB: 13.2 to 13.3 us against 13.7 to 13.8).  The
        # small cases, whose figure is the host's call rate, follow on an emptied cache.
        import torch
        big = ([bench_reduce_rotating(k, dev, "bf16") for k in (32768, 16384, 8192)] +
               [bench_reduce_rotating(k, dev, "fp32") for k in (16384, 8192)] +
               [bench_reduce_rotating(k, dev, "bf16", write_all=True) for k in (16384, 8192)] +
               [bench_reduce_rotating(k, dev, "bf16", accumulate="bf16") for k in (8192,)] +
               [bench_reduce_rotating(k, dev, "bf16", barrier=True) for k in (32768, 16384, 8192)] +
               [bench_reduce_rotating(k, dev, "fp32", barrier=True) for k in (16384, 8192)])
        torch.cuda.empty_cache()
        small = ([bench_reduce_rotating(k, dev, "bf16") for k in (16, 64, 256, 1024, 2048, 4096)] +
                 [bench_reduce_rotating(k, dev, "fp32") for k in (1024,)] +
                 [bench_reduce_rotating(k, dev, "bf16", write_all=True) for k in (1024,)] +
                 [bench_reduce_rotating(k, dev, "bf16", barrier=True) for k in (16, 1024)])
        extra["reduce_rotating"] = sorted(small + big, key=lambda r: (r["mode"], r["accumulate"], r["dtype"], r["size_kib"]))
        extra["all_gather_matmul"] = bench_ag_matmul(dev)
        extra["all_gather_matmul"]["mfma_only"] = bench_mfma_only(dev)
        extra["all_gather_matmul_fp8"] = bench_ag_matmul_fp8(dev)
        extra["gemv_allreduce"] = bench_gemv(dev)
        extra["barrier"] = bench_barrier(dev)
        try:
            extra["reduce_reference_point"] = bench_reference_point(dev)
        except Exception as exc:                    # the profiler is optional equipment
            extra["reduce_reference_point"] = {"error": repr(exc)[:200]}
    line["extra"] = extra
    line["cpu_baseline"] = cpu_baseline(args.cpu_seconds) if args.cpu_seconds > 0 else None
    print(json.dumps(line))


if __name__ == "__main__":
    main()
