"""Blockwise barrier and the host-callable halves of the signal-pad protocol.

``barrier_test`` is the drop-in for the reference's launcher
(symm_mem_recipes/triton_barrier.py:165-170).  The device function
``blockwise_barrier`` (:50-153) lives in the library's HIP code; Python cannot
call device functions, so ``blockwise_barrier`` here launches it on a grid, and
``send_signal`` / ``wait_signal`` launch one-workgroup kernels around the two
halves (:119-129 and symm_mem_recipes/triton_all_gather_matmul.py:72-95).
"""
from __future__ import annotations

import torch

from . import _lib
from .symm_mem import EmulatedSymmetricMemory


def _stream(device) -> int:
    return torch.cuda.current_stream(device).cuda_stream


def blockwise_barrier(symm_mem: EmulatedSymmetricMemory, num_blocks: int, rounds: int = 1,
                      all_ranks: bool = True, order_memory: bool = True) -> None:
    """Run ``rounds`` barrier rounds on ``num_blocks`` blocks.  With
    ``all_ranks`` every emulated rank takes part in one launch; otherwise only
    ``symm_mem.rank`` runs and its peers must be running on other streams.
    ``order_memory`` keeps the reference's release/acquire around every round;
    without it only the flags are exchanged."""
    assert num_blocks * symm_mem.world_size * 4 <= symm_mem.signal_pad_size, "signal pad too small"
    lib = _lib.load()
    rc = lib.smr_barrier(symm_mem.signal_pad_ptrs_dev, -1 if all_ranks else symm_mem.rank,
                         symm_mem.world_size, int(num_blocks), int(rounds), int(order_memory),
                         symm_mem.status.data_ptr(), _stream(symm_mem.device))
    _lib.check(rc, "blockwise_barrier")


def barrier_test(symm_mem: EmulatedSymmetricMemory) -> None:
    """32 blocks, one round, all emulated ranks (triton_barrier.py:165-170)."""
    blockwise_barrier(symm_mem, 32, 1, all_ranks=True)


def send_signal(addr: int, symm_mem: EmulatedSymmetricMemory) -> None:
    """Release-CAS 0 -> 1 on the flag at device address ``addr``."""
    _lib.check(_lib.load().smr_send_signal(int(addr), symm_mem.status.data_ptr(),
                                           _stream(symm_mem.device)), "send_signal")


def wait_signal(addr: int, symm_mem: EmulatedSymmetricMemory, reset: bool = False) -> None:
    """Wait until the flag at ``addr`` is 1 (acquire).  ``reset`` consumes it
    (CAS 1 -> 0) as the barrier's wait half does."""
    lib = _lib.load()
    fn = lib.smr_wait_signal_reset if reset else lib.smr_wait_signal
    _lib.check(fn(int(addr), symm_mem.status.data_ptr(), _stream(symm_mem.device)), "wait_signal")


def main() -> None:
    """The reference's self-check (triton_barrier.py:172-200): one barrier on 32
    blocks over zeroed 4096-word buffers must return, and the buffer prints as
    zeros.  Run as ``python -m symm_mem_recipes.barrier``."""
    import os

    world_size = int(os.environ.get("WORLD_SIZE", "8"))
    device = torch.device("cuda:0")
    torch.cuda.set_device(device)

    t = EmulatedSymmetricMemory.empty_strided_p2p(
        size=(4096,), stride=(1,), dtype=torch.uint32, device=device, world_size=world_size).fill_(0)
    symm_mem = EmulatedSymmetricMemory.rendezvous(t)
    barrier_test(symm_mem)
    torch.cuda.synchronize(device)
    symm_mem.check_status()
    print(t)


if __name__ == "__main__":
    main()
