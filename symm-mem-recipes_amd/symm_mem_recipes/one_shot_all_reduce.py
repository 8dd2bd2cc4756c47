"""One-shot all-reduce on the emulated symmetric buffers.

Drop-in for ``one_shot_all_reduce(tensor)`` of the reference
(symm_mem_recipes/triton_one_shot_all_reduce.py:96-125): same validation, same
ownership (a fresh output tensor is returned), same launch stream.  The kernel
is the library's HIP one; there is no other path.
"""
from __future__ import annotations

import torch

from . import _lib
from .symm_mem import EmulatedSymmetricMemory

NUMEL_PER_THREAD = {torch.bfloat16: 8, torch.float32: 4}      # one 128-bit slot
_DTYPE_CODE = {torch.bfloat16: _lib.DTYPE_BF16, torch.float32: _lib.DTYPE_FP32}


def num_blocks(numel: int, dtype: torch.dtype = torch.bfloat16) -> int:
    """Workgroups (= barrier blocks per rank) launched for a message; the
    counterpart of the grid formula at triton_one_shot_all_reduce.py:106-109."""
    return _lib.load().smr_reduce_num_blocks(int(numel), _DTYPE_CODE[dtype])


def one_shot_all_reduce(tensor: torch.Tensor, *, barrier: bool = True, write_all: bool = False,
                        all_ranks: bool = False, accumulate: str = "fp32",
                        trailing_barrier: bool = False, device_table: bool = False) -> torch.Tensor:
    """Sum the symmetric buffers of all ranks element-wise (fp32 accumulator,
    rank order 0..world_size-1) and return the calling rank's result.

    ``barrier``    run the blockwise handshake before reading the peers
                   (triton_one_shot_all_reduce.py:70); the other ranks' halves
                   are played by spare lanes of the wave that does the rank's own.
    ``write_all``  write the result back into all peer buffers in place and
                   return the calling rank's buffer (``tensor`` itself).
    ``all_ranks``  run every emulated rank in one launch, each behind the real
                   barrier; returns ``[world_size, *tensor.shape]``.
                   Together with ``write_all`` it is the two-shot all-reduce:
                   rank r reduces the r-th slice only and writes it into every
                   peer's buffer, between two handshakes; returns the
                   ``[world_size, *tensor.shape]`` view of the buffers.
    ``trailing_barrier`` a second handshake after the last store (the reference
                   has none behind triton_one_shot_all_reduce.py:93): no peer
                   can overwrite its buffer while another still reads it.
    ``device_table`` let the kernel read the peers' buffer and signal pad addresses from the
                   tables in device memory, as the reference's does
                   (triton_one_shot_all_reduce.py:86-87, triton_barrier.py:100-110); by default
                   they are passed as kernel arguments, which saves a dependent load in front
                   of the handshake and another in front of the first data load.
    ``accumulate`` "fp32" (default) keeps an fp32 accumulator and rounds once;
                   "bf16" rounds the accumulator to bf16 after every add, which is
                   bit for bit the reference's add.bf16x2 chain
                   (triton_one_shot_all_reduce.py:36-49, 84-89); bf16 tensors only.
    """
    # Calls after the first for one (buffer, size, options) take the prepared launch: for
    # messages of a few KiB - the reference's own operating point, :146 - the host path is
    # most of a call, so the validation, the handle lookup and the argument marshalling are
    # done once per allocation and kept with it (they die with it at release()).
    key = (tensor.numel(), tensor.dtype, barrier, write_all, all_ranks, accumulate, trailing_barrier, device_table)
    entry = EmulatedSymmetricMemory._by_addr.get(tensor.data_ptr())
    launch = entry[0].launches.get((entry[1],) + key) if entry is not None else None
    if launch is None:
        launch = _prepare(tensor, entry, key)
    fn, table, pads, numel, dtype_code, rank, world_size, write_flag, barrier_mode, status, kind, device_index = launch
    if not tensor.is_contiguous():
        raise AssertionError("tensor must be contiguous")
    if kind == _OUT_NEW:
        output = torch.empty_like(tensor)
        out_ptr = output.data_ptr()
    elif kind == _OUT_ALL_RANKS:
        output = torch.empty((world_size,) + tuple(tensor.shape), dtype=tensor.dtype, device=tensor.device)
        out_ptr = output.data_ptr()
    else:
        output, out_ptr = tensor, 0
    rc = fn(table, pads, out_ptr, numel, dtype_code, rank, world_size, write_flag, barrier_mode, status,
            _raw_stream(device_index))
    if rc != 0:
        _lib.check(rc, "one_shot_all_reduce")
    if kind == _OUT_TWO_SHOT:
        return EmulatedSymmetricMemory(entry[0], entry[1]).all_buffers(tuple(tensor.shape), tensor.dtype)
    return output


_OUT_NEW, _OUT_ALL_RANKS, _OUT_IN_PLACE, _OUT_TWO_SHOT = range(4)
#: the current stream's handle without building a torch.cuda.Stream object around it
_raw_stream = torch._C._cuda_getCurrentRawStream


def _prepare(tensor: torch.Tensor, entry, key):
    """Validation (the reference's asserts, triton_one_shot_all_reduce.py:102-105,111) and the
    launch arguments that do not change from call to call, cached with the allocation."""
    _, _, barrier, write_all, all_ranks, accumulate, trailing_barrier, device_table = key
    assert accumulate in ("fp32", "bf16"), "accumulate must be 'fp32' or 'bf16'"
    assert accumulate == "fp32" or tensor.dtype == torch.bfloat16, "accumulate='bf16' needs a bfloat16 tensor"
    assert tensor.dtype in _DTYPE_CODE, "Only bfloat16 and float32 are supported for now."
    assert (
        tensor.numel() % NUMEL_PER_THREAD[tensor.dtype] == 0
    ), "The number of elements must be 128-bit aligned."
    assert tensor.is_contiguous(), "tensor must be contiguous"
    symm_mem = EmulatedSymmetricMemory.rendezvous(tensor)
    assert symm_mem is not None, "tensor must be allocated via SymmetricMemory"

    lib = _lib.load()
    two_shot = write_all and all_ranks
    if two_shot:
        assert barrier, "the two-shot form needs its handshakes"
        kind = _OUT_TWO_SHOT
    elif write_all:
        kind = _OUT_IN_PLACE
    elif all_ranks:
        kind = _OUT_ALL_RANKS
    else:
        kind = _OUT_NEW
    fn, table, pads = ((lib.smr_one_shot_all_reduce, symm_mem.buffer_ptrs_dev, symm_mem.signal_pad_ptrs_dev)
                       if device_table else
                       (lib.smr_one_shot_all_reduce_addrs, symm_mem.buffer_ptrs_host, symm_mem.signal_pad_ptrs_host))
    barrier_mode = ((_lib.BARRIER_BOTH if (trailing_barrier or two_shot) else _lib.BARRIER_PROXY) if barrier
                    else _lib.BARRIER_NONE)
    device_index = tensor.device.index if tensor.device.index is not None else torch.cuda.current_device()
    launch = (fn, table, pads, tensor.numel(),
              _lib.DTYPE_BF16_STEPWISE if accumulate == "bf16" else _DTYPE_CODE[tensor.dtype],
              -1 if all_ranks else symm_mem.rank, symm_mem.world_size, 1 if write_all else 0, barrier_mode,
              symm_mem.status.data_ptr(), kind, device_index)
    entry[0].launches[(entry[1],) + key] = launch
    return launch


def main() -> None:
    """The reference's self-check and latency line
    (triton_one_shot_all_reduce.py:128-162): 8192 ones per rank must sum to
    world_size, then the kernel's median device time.  The ranks are emulated in
    one GPU's memory (WORLD_SIZE, default 8); run as
    ``python -m symm_mem_recipes.one_shot_all_reduce``."""
    import os

    from .utils import benchmark_with_profiler

    world_size = int(os.environ.get("WORLD_SIZE", "8"))
    device = torch.device("cuda:0")
    torch.cuda.set_device(device)

    tensor = EmulatedSymmetricMemory.empty_strided_p2p(
        size=(8192,), stride=(1,), dtype=torch.bfloat16, device=device, world_size=world_size)
    symm_mem = EmulatedSymmetricMemory.rendezvous(tensor)
    for r in range(world_size):
        symm_mem.get_buffer(r, (8192,), torch.bfloat16).fill_(1)

    output = one_shot_all_reduce(tensor)
    assert output.eq(world_size).all().item()
    symm_mem.check_status()

    lat_us = benchmark_with_profiler(lambda: one_shot_all_reduce(tensor),
                                     r".*one_shot_all_reduce_kernel", benchmark_iters=200)
    print(f"Median latency: {lat_us:.2f} us")


if __name__ == "__main__":
    main()
