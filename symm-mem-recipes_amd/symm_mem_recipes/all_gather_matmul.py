"""All-gather matmul: a producer that gathers the peers' A shards and raises one
progress flag per chunk, overlapped with a bf16 GEMM that walks the shards in
their ready order and waits on those flags.

Drop-ins for the reference's host entry points
(symm_mem_recipes/triton_all_gather_matmul.py): ``all_gather_with_progress``
(:20-56), ``all_gather_matmul_tma_persistent`` (:219-319; the name is kept although
nothing here is TMA - the kernel is an LDS-staged MFMA GEMM) and the torch
comparator ``all_gather_matmul`` (:322-326).
"""
from __future__ import annotations

import ctypes
import os
from typing import Optional

import torch

from . import _lib
from .symm_mem import EmulatedSymmetricMemory, _get_backend_stream

#: Flags, tickets and counters of the fused launch, one array per (device, stream, size): the
#: kernel leaves it zeroed, so it is filled once when it is made and never again.
_fused_state = {}


def _state_for(device: torch.device, stream: int, words: int) -> torch.Tensor:
    if torch.cuda.is_current_stream_capturing():
        # memory allocated under capture belongs to the graph: a fresh array, whose fill is
        # recorded with the launch (a fill kernel, replayed with it), and nothing cached
        return torch.zeros(words, dtype=torch.int32, device=device)
    key = (device.index, int(stream), int(words))
    st = _fused_state.get(key)
    if st is None:
        st = torch.zeros(words, dtype=torch.int32, device=device)
        _fused_state[key] = st
    return st


def all_gather_with_progress(output: torch.Tensor, inp: torch.Tensor, progress: torch.Tensor,
                             splits_per_rank: int, num_workgroups: int = 0) -> None:
    """Copy every rank's shard into ``output`` (sources in the order rank+1, ...,
    rank+world_size-1, rank) and set ``progress[src*splits_per_rank + split]`` to 1
    after each chunk, on the current stream."""
    assert inp.is_contiguous()

    symm_mem = EmulatedSymmetricMemory.rendezvous(inp)
    assert symm_mem is not None

    rank = symm_mem.rank
    world_size = symm_mem.world_size

    assert inp.numel() % splits_per_rank == 0
    assert progress.numel() == world_size * splits_per_rank
    assert progress.element_size() == 4 and progress.is_contiguous()

    output_shape = list(inp.shape)
    output_shape[0] *= world_size
    assert list(output.shape) == output_shape, (list(output.shape), output_shape)
    assert output.is_contiguous() and output.dtype == inp.dtype

    counters = torch.zeros(world_size * splits_per_rank, dtype=torch.int32, device=inp.device)
    _launch_producer(symm_mem, output, inp, progress, counters, splits_per_rank, num_workgroups,
                     torch.cuda.current_stream(inp.device).cuda_stream)
    symm_mem.barrier()


def _launch_producer(symm_mem, output, inp, progress, counters, splits_per_rank, num_workgroups,
                     stream_handle, at_once: bool = False) -> None:
    """The producer kernel on the given stream; ``counters`` (one zeroed int32 per
    chunk) are its arrival counters.  ``at_once`` copies all chunks together and raises
    the flags at the end, for a consumer that is queued behind the copy."""
    lib = _lib.load()
    rc = (lib.smr_all_gather_at_once if at_once else lib.smr_all_gather_with_progress)(
        symm_mem.buffer_ptrs_dev, output.data_ptr(), progress.data_ptr(), counters.data_ptr(),
        symm_mem.rank, symm_mem.world_size, inp.numel() * inp.element_size(), int(splits_per_rank),
        int(num_workgroups), stream_handle)
    _lib.check(rc, "all_gather_with_progress")


def all_gather_matmul_tma_persistent(a_shard: torch.Tensor, b: torch.Tensor, a_out: torch.Tensor,
                                     c_out: torch.Tensor, configs: Optional[dict] = None,
                                     mm_only: bool = False, *, splits_per_rank: int = 1,
                                     fused=None, producer_workgroups: Optional[int] = None,
                                     check: bool = False) -> torch.Tensor:
    """``c_out = cat(all ranks' a_shard) @ b.T`` with ``b`` of shape [N, K]
    (K-contiguous), bf16 or - all four tensors - float8_e4m3fn.  ``mm_only`` skips the gather and the flags and multiplies
    what ``a_shard`` (rank 0's rows) and ``a_out`` already hold: the ungated
    comparator.  ``configs`` is accepted for compatibility; the tile shape is the
    library's choice.

    Keyword arguments beyond the reference's signature (triton_all_gather_matmul.py:219-221):
    ``fused``      None: the library's plan decides between the fused launch and, for a GEMM too
                   short to hide the copy behind, copy-then-multiply; True / False force one.
                   "streams": the reference's own choreography (:246-253, 318) - fresh zeroed
                   flags, the stand-alone producer on the backend stream, the GEMM on the
                   current stream gated on flags that the producer raises, stream join.
    ``producer_workgroups`` copy-only workgroups of the fused launch (workgroups of the producer
                   kernel with "streams"); None = the plan's.
    ``check``      synchronise and raise if a bounded wait inside the kernel expired (the result
                   is then not valid); without it the caller looks at ``check_status()`` later.
    """
    if mm_only:
        symm_mem = None
        rank = 0
        world_size = int(os.environ.get("WORLD_SIZE", "8"))
    else:
        symm_mem = EmulatedSymmetricMemory.rendezvous(a_shard)
        assert symm_mem is not None, "a_shard must be allocated via SymmetricMemory"
        rank = symm_mem.rank
        world_size = symm_mem.world_size

    # bf16, or e4m3fn throughout as the reference's FP8_OUTPUT switch (:115,123,311)
    fp8 = a_shard.dtype == torch.float8_e4m3fn
    assert a_shard.dtype in (torch.bfloat16, torch.float8_e4m3fn), "Only bfloat16 and float8_e4m3fn are supported."
    assert b.dtype == a_shard.dtype and a_out.dtype == a_shard.dtype and c_out.dtype == a_shard.dtype, \
        "a_shard, b, a_out and c_out must have one dtype"
    M = a_shard.shape[0] * world_size
    N = b.shape[0]
    K = a_shard.shape[1]

    assert fused in (None, True, False, "streams"), "fused must be None, True, False or 'streams'"
    assert b.shape[1] == K
    assert a_out.shape[0] == M
    assert a_out.shape[1] == K
    assert c_out.shape[0] == M
    assert c_out.shape[1] == N
    assert a_shard.is_contiguous() and b.is_contiguous() and a_out.is_contiguous() and c_out.is_contiguous()

    COMM_BLOCK_SIZE_M = M // world_size // splits_per_rank
    if configs is not None and "BLOCK_SIZE_M" in configs:
        assert COMM_BLOCK_SIZE_M % (configs["BLOCK_SIZE_M"] * configs.get("GROUP_SIZE_M", 1)) == 0

    lib = _lib.load()
    device = a_shard.device
    current = torch.cuda.current_stream(device)
    status_ptr = symm_mem.status.data_ptr() if symm_mem is not None else 0
    gemm = lib.smr_ag_matmul_fp8 if fp8 else lib.smr_ag_matmul

    if mm_only:
        rc = gemm(a_shard.data_ptr(), a_out.data_ptr(), b.data_ptr(), c_out.data_ptr(), 0, M, N, K, rank,
                  world_size, COMM_BLOCK_SIZE_M, 0, status_ptr, current.cuda_stream)
        _lib.check(rc, "all_gather_matmul")
        return c_out

    symm_mem.barrier(0)
    plan = (ctypes.c_int32 * 5)()
    planner = lib.smr_ag_matmul_plan_fp8 if fp8 else lib.smr_ag_matmul_plan
    _lib.check(planner(M, N, K, world_size, COMM_BLOCK_SIZE_M, plan), "all_gather_matmul")
    sequential = bool(plan[4]) if fused is None else not fused
    chunks = world_size * splits_per_rank
    state = None
    if fused == "streams":
        # The reference's form: `progress` starts at zero, the producer runs on the backend
        # stream behind everything queued so far, the GEMM on the current stream waits for each
        # chunk's flag, and the current stream joins the backend stream at the end.  For bf16 the
        # producer is the one whose workgroups fit beside the GEMM's on the same compute units
        # (smr_all_gather_beside: it costs no compute units, like the reference's copy engines),
        # and the GEMM takes the whole GPU.  The widest e4m3fn tile leaves no registers for a
        # neighbour: there the producer gets compute units of its own and the GEMM's grid leaves
        # them free.  Every wait inside the GEMM is bounded.
        flags = torch.zeros(2 * chunks, dtype=torch.int32, device=device)     # progress, arrival counters
        backend_stream = _get_backend_stream()
        flags.record_stream(backend_stream)
        backend_stream.wait_stream(current)
        beside = not fp8
        producer = lib.smr_all_gather_beside if beside else lib.smr_all_gather_with_progress
        wgs = (0 if beside else int(plan[1])) if producer_workgroups is None else int(producer_workgroups)
        args = [symm_mem.buffer_ptrs_dev, a_out.data_ptr(), flags.data_ptr(), flags[chunks:].data_ptr(),
                rank, world_size, a_shard.numel() * a_shard.element_size(), int(splits_per_rank), wgs]
        if beside:
            # its timetable: the first pass's ranks flat out, the others as the GEMM gets to them
            # (a GEMM shorter than the copy gets everything flat out whatever the estimate says)
            pace = (ctypes.c_int32 * 2)()
            _lib.check(lib.smr_ag_matmul_pace(M, N, K, world_size, COMM_BLOCK_SIZE_M, 2, pace), "all_gather_matmul")
            args += [int(pace[0]), int(pace[1])]
        rc = producer(*args, backend_stream.cuda_stream)
        _lib.check(rc, "all_gather_with_progress")
        rc = gemm(a_shard.data_ptr(), a_out.data_ptr(), b.data_ptr(), c_out.data_ptr(), flags.data_ptr(), M, N, K,
                  rank, world_size, COMM_BLOCK_SIZE_M, int(beside), status_ptr, current.cuda_stream)
        current.wait_stream(backend_stream)
    elif sequential:
        # Too small to hide the copy behind the GEMM: the whole GPU copies, then the whole
        # GPU multiplies, in stream order (the GEMM then needs no flags).
        scratch = torch.zeros(2 * chunks, dtype=torch.int32, device=device)
        wide = torch.cuda.get_device_properties(device).multi_processor_count
        _launch_producer(symm_mem, a_out, a_shard, scratch[:chunks], scratch[chunks:], splits_per_rank, wide,
                         current.cuda_stream, at_once=True)
        rc = gemm(a_shard.data_ptr(), a_out.data_ptr(), b.data_ptr(), c_out.data_ptr(), 0, M, N, K, rank,
                  world_size, COMM_BLOCK_SIZE_M, 0, status_ptr, current.cuda_stream)
    else:
        # One launch on the current stream: GEMM workgroups and copy-only workgroups in one
        # grid, flags in an array the kernel itself leaves zeroed (no fill, no second stream;
        # the reference needs both, :249-253,318, because its producer is a copy engine).
        state = _state_for(device, current.cuda_stream, lib.smr_ag_matmul_fused_state_words(world_size, splits_per_rank))
        rc = lib.smr_ag_matmul_fused(
            a_shard.data_ptr(), a_out.data_ptr(), b.data_ptr(), c_out.data_ptr(), state.data_ptr(),
            symm_mem.buffer_ptrs_dev, 1 if fp8 else 2, M, N, K, rank, world_size, COMM_BLOCK_SIZE_M,
            0 if producer_workgroups is None else int(producer_workgroups), status_ptr, current.cuda_stream)
    _lib.check(rc, "all_gather_matmul")
    if check:
        try:
            symm_mem.check_status()
        except _lib.SmrError:
            if state is not None:
                state.zero_()          # a launch that gave up leaves flags and tickets behind
            raise
    return c_out


#: the same entry point under a name that says what it is
all_gather_matmul_fused = all_gather_matmul_tma_persistent


def all_gather_matmul(a_shard: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
    """The unfused comparator: gather the shards, then one library matmul
    (triton_all_gather_matmul.py:322-326; ``b`` is [K, N] here, as there)."""
    symm_mem = EmulatedSymmetricMemory.rendezvous(a_shard)
    assert symm_mem is not None, "a_shard must be allocated via SymmetricMemory"
    a = torch.cat([symm_mem.get_buffer(r, a_shard.shape, a_shard.dtype)
                   for r in range(symm_mem.world_size)], dim=0)
    return torch.matmul(a, b)


def gemm_schedule(M: int, N: int, K: int, rank: int, world_size: int, comm_block_m: int,
                  gated=True):
    """The tile order the GEMM uses on a 256-CU part, as a list of dicts in each
    workgroup's visiting order (host-only; the counterpart of the index
    arithmetic at triton_all_gather_matmul.py:125-174).  ``gated``: False / 0 an ungated
    launch, True / 1 a gated one that leaves compute units to a producer kernel, 2 a gated one
    that takes the whole GPU (``whole_gpu`` of smr_ag_matmul)."""
    import ctypes
    lib = _lib.load()
    n = lib.smr_ag_matmul_schedule(M, N, K, rank, world_size, comm_block_m, int(gated), None, 0)
    if n < 0:
        _lib.check(n, "gemm_schedule")
    buf = (ctypes.c_int32 * (8 * n))()
    lib.smr_ag_matmul_schedule(M, N, K, rank, world_size, comm_block_m, int(gated), buf, n)
    keys = ("wg", "step", "row0", "col0", "rows", "cols", "comm_block", "local")
    return [dict(zip(keys, buf[8 * i:8 * i + 8])) for i in range(n)]


def main(argv=None) -> None:
    """The reference's harness (triton_all_gather_matmul.py:329-418) with its
    options (all but --print_ptx: there is no PTX): fused result checked against gather + library matmul, then the four
    latency lines.  The tile options are accepted and checked as there
    (rows per flag must divide into BLOCK_SIZE_M * GROUP_SIZE_M); the tile the
    kernel runs is the library's.  Run as ``python -m symm_mem_recipes.all_gather_matmul``."""
    import argparse

    from .utils import benchmark_with_event

    ap = argparse.ArgumentParser(description="all-gather matmul: parity check and latencies")
    ap.add_argument("--M", type=int, default=4096)
    ap.add_argument("--N", type=int, default=6656)
    ap.add_argument("--K", type=int, default=16384)
    ap.add_argument("--BLOCK_SIZE_M", type=int, default=128)
    ap.add_argument("--BLOCK_SIZE_N", type=int, default=256)
    ap.add_argument("--BLOCK_SIZE_K", type=int, default=64)
    ap.add_argument("--GROUP_SIZE_M", type=int, default=4)
    ap.add_argument("--num_stages", type=int, default=3)
    ap.add_argument("--num_warps", type=int, default=8)
    args = ap.parse_args(argv)

    rank = int(os.environ.get("RANK", "0"))
    world_size = int(os.environ.get("WORLD_SIZE", "8"))
    device = torch.device("cuda:0")
    torch.cuda.set_device(device)
    m, n, k = args.M, args.N, args.K

    a_shard = EmulatedSymmetricMemory.empty_strided_p2p(
        size=(m // world_size, k), stride=(k, 1), dtype=torch.bfloat16, device=device,
        world_size=world_size, rank=rank)
    symm_mem = EmulatedSymmetricMemory.rendezvous(a_shard)
    for r in range(world_size):
        torch.manual_seed(42 + r)
        symm_mem.get_buffer(r, (m // world_size, k), torch.bfloat16).normal_()
    torch.manual_seed(42 + rank)
    a = torch.randn((m, k), device=device, dtype=torch.bfloat16)
    b = torch.randn((k, n), device=device, dtype=torch.bfloat16).T.contiguous()
    c = torch.randn((m, n), device=device, dtype=torch.bfloat16)

    configs = {
        "BLOCK_SIZE_M": args.BLOCK_SIZE_M, "BLOCK_SIZE_N": args.BLOCK_SIZE_N,
        "BLOCK_SIZE_K": args.BLOCK_SIZE_K, "GROUP_SIZE_M": args.GROUP_SIZE_M,
        "num_stages": args.num_stages, "num_warps": args.num_warps,
    }

    c0 = all_gather_matmul(a_shard, b.T)
    c1 = all_gather_matmul_tma_persistent(a_shard, b, a, c, configs)
    symm_mem.check_status()
    # two GEMMs that sum K in different orders: bf16's last place (2^-8) of the larger of the
    # two values is what can differ, plus cancellation noise relative to the row's magnitude
    assert torch.allclose(c0.float(), c1.float(), rtol=1e-2, atol=1e-2 * c0.float().abs().max().item())

    lat_us = benchmark_with_event(lambda: torch.matmul(a, b.T, out=c), flush_l2=True)
    print(f"library matmul only: {lat_us} us")
    lat_us = benchmark_with_event(
        lambda: all_gather_matmul_tma_persistent(a_shard, b, a, c, configs, mm_only=True), flush_l2=True)
    print(f"hip matmul only: {lat_us} us")
    lat_us = benchmark_with_event(lambda: all_gather_matmul(a_shard, b.T), flush_l2=True)
    print(f"library gather + matmul: {lat_us} us")
    lat_us = benchmark_with_event(
        lambda: all_gather_matmul_tma_persistent(a_shard, b, a, c, configs), flush_l2=True)
    print(f"hip all_gather_matmul: {lat_us} us")
    symm_mem.check_status()
    # the reference's own choreography: producer on the backend stream, GEMM gated on its flags
    c2 = torch.empty_like(c)
    all_gather_matmul_tma_persistent(a_shard, b, a, c2, configs, fused="streams")
    symm_mem.check_status()
    assert torch.equal(c1.view(torch.int16), c2.view(torch.int16))
    lat_us = benchmark_with_event(
        lambda: all_gather_matmul_tma_persistent(a_shard, b, a, c, configs, fused="streams"), flush_l2=True)
    print(f"hip all_gather_matmul, producer on a second stream: {lat_us} us")
    symm_mem.check_status()


if __name__ == "__main__":
    main()
