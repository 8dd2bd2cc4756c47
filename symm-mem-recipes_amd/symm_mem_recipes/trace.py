"""Timeline of one all-gather matmul launch from the kernels' own time stamps.

The library's kernels can write time stamps of the GPU's 100 MHz clock into a
registered buffer (``smr_set_trace_buffer``): when the producer started and raised each
flag, and for every GEMM workgroup and tile when the tile was picked, when its flag wait
was over, when its K loop ended and when it was stored.  This module runs a launch with
the buffer registered and prints the summary; the reference's counterpart is its
profiler hook (symm_mem_recipes/utils.py:41-52).

    python -m symm_mem_recipes.trace --M 16384 --N 3584 --K 8192
"""
from __future__ import annotations

import argparse
import importlib
import statistics

import torch

from . import _lib
from .symm_mem import EmulatedSymmetricMemory

PRODUCER_WORDS = 64
STEPS = 16
GEMM_WORDS = 256 * STEPS * 4
TICKS_PER_US = 100.0


def trace_launch(M: int, N: int, K: int, mode: str = "fused", world_size: int = 8, rank: int = 0,
                 warm: int = 20, device=None, dtype: torch.dtype = torch.bfloat16) -> dict:
    """Run ``warm`` launches and return the time stamps of the last one, in microseconds from
    the first workgroup's entry.  ``mode``: "ungated", "fused" (the library's default launch),
    "streams" (the reference's choreography: stand-alone producer on the backend stream, GEMM
    gated on its flags) or "sequential" (copy-then-multiply).

    Returns ``{"end_us", "producer_start_us", "flags_us": {chunk: t}, "steps": [per-step dict]}``;
    a step holds the medians over the workgroups of: start, wait (flag wait, with the copying
    done meanwhile), k_loop, store, and the time the slowest workgroup stored the tile."""
    agm = importlib.import_module(__package__ + ".all_gather_matmul")
    lib = _lib.load()
    device = torch.device("cuda:0") if device is None else device
    std = 0.05 if dtype == torch.float8_e4m3fn else 0.02
    a_shard = EmulatedSymmetricMemory.empty_strided_p2p((M // world_size, K), (K, 1), dtype, device,
                                                        world_size=world_size, rank=rank)
    h = EmulatedSymmetricMemory.rendezvous(a_shard)
    g = torch.Generator(device=device)
    for r in range(world_size):
        g.manual_seed(42 + r)
        h.get_buffer(r, (M // world_size, K), dtype).copy_(
            torch.empty(M // world_size, K, device=device).normal_(0, std, generator=g).to(dtype))
    b = torch.empty(N, K, device=device).normal_(0, std, generator=g).to(dtype)
    a_out = torch.cat([h.get_buffer(r, (M // world_size, K), dtype) for r in range(world_size)])
    c = torch.empty(M, N, dtype=torch.uint8 if dtype == torch.float8_e4m3fn else dtype, device=device).view(dtype)
    flush = torch.empty(1 << 28, dtype=torch.int32, device=device)
    words = PRODUCER_WORDS + GEMM_WORDS
    trace = torch.zeros(words, dtype=torch.int64, device=device)

    kwargs = {"fused": {"sequential": False, "ungated": None, "streams": "streams"}.get(mode, True)}
    try:
        _lib.check(lib.smr_set_trace_buffer(trace.data_ptr(), words), "trace")
        for _ in range(warm):
            flush.zero_()
            agm.all_gather_matmul_tma_persistent(a_shard, b, a_out, c, None, mm_only=(mode == "ungated"), **kwargs)
        torch.cuda.synchronize(device)
        h.check_status()
    finally:
        lib.smr_set_trace_buffer(None, 0)
        EmulatedSymmetricMemory.release(a_shard)

    t = trace.cpu().tolist()
    stamps = [[t[PRODUCER_WORDS + (wg * STEPS + s) * 4:PRODUCER_WORDS + (wg * STEPS + s) * 4 + 4]
               for s in range(STEPS)] for wg in range(256)]
    starts = [st[0][0] for st in stamps if st[0][0] > 0]
    t0 = min(starts)
    us = lambda ticks: (ticks - t0) / TICKS_PER_US
    out = {"mode": mode, "steps": [], "flags_us": {}, "producer_start_us": None}
    if mode in ("fused", "streams"):
        out["producer_start_us"] = us(t[PRODUCER_WORDS - 1])
        chunks = world_size * 1
        out["flags_us"] = {i: us(t[i]) for i in range(chunks) if t[i] > t0}
    end = 0.0
    for s in range(STEPS):
        rows = [st[s] for st in stamps if st[s][0] > 0 and st[s][3] > 0]
        if not rows:
            continue
        med = statistics.median
        out["steps"].append({
            "step": s, "workgroups": len(rows),
            "start_us": med(us(r[0]) for r in rows),
            "wait_us": med((r[1] - r[0]) / TICKS_PER_US for r in rows),
            "k_loop_us": med((r[2] - r[1]) / TICKS_PER_US for r in rows),
            "store_us": med((r[3] - r[2]) / TICKS_PER_US for r in rows),
            "last_stored_us": max(us(r[3]) for r in rows),
        })
        end = max(end, out["steps"][-1]["last_stored_us"])
    out["end_us"] = end
    return out


def main(argv=None) -> None:
    ap = argparse.ArgumentParser(description=__doc__.split("\n\n")[0])
    ap.add_argument("--M", type=int, default=16384)
    ap.add_argument("--N", type=int, default=3584)
    ap.add_argument("--K", type=int, default=8192)
    ap.add_argument("--fp8", action="store_true")
    ap.add_argument("--modes", default="ungated,fused,streams")
    args = ap.parse_args(argv)
    dtype = torch.float8_e4m3fn if args.fp8 else torch.bfloat16
    for mode in args.modes.split(","):
        r = trace_launch(args.M, args.N, args.K, mode, dtype=dtype)
        print(f"## {mode}: last tile stored {r['end_us']:.1f} us after the first workgroup's entry")
        if r["producer_start_us"] is not None:
            flags = ", ".join(f"{i}: {v:.0f}" for i, v in sorted(r["flags_us"].items(), key=lambda kv: kv[1]))
            print(f"producer starts at {r['producer_start_us']:.1f} us; flags raised at (chunk: us) {flags}")
        print("| step | workgroups | start (median us) | wait | K loop | epilogue | last workgroup stored at |")
        print("|---|---|---|---|---|---|---|")
        for s in r["steps"]:
            print(f"| {s['step']} | {s['workgroups']} | {s['start_us']:.1f} | {s['wait_us']:.1f} | "
                  f"{s['k_loop_us']:.1f} | {s['store_us']:.1f} | {s['last_stored_us']:.1f} |")
        print(flush=True)


if __name__ == "__main__":
    main()
