"""Single-GPU emulation of the symmetric-memory handle the recipes are written
against (torch's ``_SymmetricMemory``; call sites in the reference:
symm_mem_recipes/triton_one_shot_all_reduce.py:111-120,145-151,
symm_mem_recipes/triton_barrier.py:167-169,190-198,
symm_mem_recipes/triton_all_gather_matmul.py:28-32,46-56,226-229,250).

One allocation holds the buffers of all ``world_size`` emulated ranks back to back
in the HBM of one MI355X, together with one zero-initialised signal pad per rank
and the two device pointer tables (``buffer_ptrs_dev``, ``signal_pad_ptrs_dev``)
that the kernels index by rank.  ``empty_strided_p2p`` returns the calling
rank's view of it; ``rendezvous`` maps a view back to its handle.  The calling
rank is process-wide state (``set_rank``), since one process plays every rank.
"""
from __future__ import annotations

import ctypes
import math
import os
from typing import Dict, List, Optional, Sequence, Tuple

import torch

from . import _lib

#: bytes per emulated signal pad: 4096 blocks x 8 ranks x 4 B
SIGNAL_PAD_SIZE = 128 * 1024
_ALIGN = 256
_STAGGER = 4096        # bytes between the end of one rank's buffer and the start of the next

_current_rank = int(os.environ.get("RANK", "0"))
_default_world_size = int(os.environ.get("WORLD_SIZE", "8"))


def set_rank(rank: int) -> None:
    """Select which emulated rank subsequent ``empty_strided_p2p`` calls speak for."""
    global _current_rank
    _current_rank = int(rank)


def get_rank() -> int:
    return _current_rank


def set_world_size(world_size: int) -> None:
    global _default_world_size
    assert 1 <= world_size <= _lib.MAX_WORLD_SIZE
    _default_world_size = int(world_size)


def get_world_size() -> int:
    return _default_world_size


class _Group:
    """One symmetric allocation: ws buffers, ws pads, pointer tables, status words."""

    def __init__(self, nbytes: int, device: torch.device, world_size: int):
        self.world_size = world_size
        self.device = device
        self.buffer_size = max(_ALIGN, (nbytes + _ALIGN - 1) // _ALIGN * _ALIGN)
        # Peers' buffers one GPU apart would share no DRAM; emulated in one slab, eight read
        # streams that are congruent modulo a power of two keep landing in the same banks
        # (8 x 16 MiB reduce: 27.5 us; staggered by 4 KiB per rank: 25.5 us).
        self.buffer_stride = self.buffer_size + _STAGGER
        self.slab = torch.empty(world_size * self.buffer_stride, dtype=torch.uint8, device=device)
        self.pads = torch.zeros(world_size * SIGNAL_PAD_SIZE, dtype=torch.uint8, device=device)
        base = self.slab.data_ptr()
        pbase = self.pads.data_ptr()
        self.buffer_addrs = [base + r * self.buffer_stride for r in range(world_size)]
        self.pad_addrs = [pbase + r * SIGNAL_PAD_SIZE for r in range(world_size)]
        # the same addresses as a host array, for entry points that take them by value
        self.buffer_addrs_host = (ctypes.c_uint64 * _lib.MAX_WORLD_SIZE)(*self.buffer_addrs)
        self.pad_addrs_host = (ctypes.c_uint64 * _lib.MAX_WORLD_SIZE)(*self.pad_addrs)
        self.buffer_ptrs = torch.tensor(self.buffer_addrs, dtype=torch.int64, device=device)
        self.pad_ptrs = torch.tensor(self.pad_addrs, dtype=torch.int64, device=device)
        self.status = torch.zeros(_lib.STATUS_WORDS, dtype=torch.int32, device=device)
        #: prepared launches of the entry points, keyed by (rank, size, options); they hold
        #: addresses of this allocation and go with it
        self.launches: Dict[tuple, tuple] = {}


class EmulatedSymmetricMemory:
    """Per-rank handle; mirrors the attributes and methods of ``_SymmetricMemory``
    that the recipes use."""

    _by_addr: Dict[int, Tuple[_Group, int]] = {}

    def __init__(self, group: _Group, rank: int):
        self._group = group
        self.rank = rank
        self.world_size = group.world_size
        self.buffer_size = group.buffer_size
        self.signal_pad_size = SIGNAL_PAD_SIZE
        self.device = group.device

    # ---- pointer tables, as integer device addresses (what the kernels take)
    @property
    def buffer_ptrs_dev(self) -> int:
        return self._group.buffer_ptrs.data_ptr()

    @property
    def signal_pad_ptrs_dev(self) -> int:
        return self._group.pad_ptrs.data_ptr()

    @property
    def buffer_ptrs_host(self):
        """ctypes array of the ranks' buffer addresses in host memory."""
        return self._group.buffer_addrs_host

    @property
    def signal_pad_ptrs_host(self):
        """ctypes array of the ranks' signal pad addresses in host memory."""
        return self._group.pad_addrs_host

    @property
    def buffer_ptrs(self) -> List[int]:
        return list(self._group.buffer_addrs)

    @property
    def signal_pad_ptrs(self) -> List[int]:
        return list(self._group.pad_addrs)

    # ---- allocation / lookup
    @staticmethod
    def empty_strided_p2p(size: Sequence[int], stride: Sequence[int], dtype: torch.dtype,
                          device, group_name: Optional[str] = None, *,
                          world_size: Optional[int] = None, rank: Optional[int] = None) -> torch.Tensor:
        size = tuple(int(s) for s in size)
        stride = tuple(int(s) for s in stride)
        device = torch.device(device)
        ws = _default_world_size if world_size is None else int(world_size)
        rank = _current_rank if rank is None else int(rank)
        assert 1 <= ws <= _lib.MAX_WORLD_SIZE, "world_size must be 1..8"
        assert 0 <= rank < ws, "rank out of range"
        assert len(size) == len(stride)
        span = 1 + sum((n - 1) * s for n, s in zip(size, stride)) if all(n > 0 for n in size) else 0
        itemsize = torch.empty((), dtype=dtype).element_size()
        group = _Group(span * itemsize, device, ws)
        for r in range(ws):
            EmulatedSymmetricMemory._by_addr[group.buffer_addrs[r]] = (group, r)
        return EmulatedSymmetricMemory(group, rank)._view(rank, size, stride, dtype, 0)

    @staticmethod
    def rendezvous(tensor: torch.Tensor) -> Optional["EmulatedSymmetricMemory"]:
        entry = EmulatedSymmetricMemory._by_addr.get(tensor.data_ptr())
        if entry is None:
            return None
        group, rank = entry
        return EmulatedSymmetricMemory(group, rank)

    @staticmethod
    def release(tensor: Optional[torch.Tensor] = None) -> None:
        """Drop the registry's reference to one allocation (or to all of them)."""
        reg = EmulatedSymmetricMemory._by_addr
        if tensor is None:
            reg.clear()
            return
        entry = reg.get(tensor.data_ptr())
        if entry is not None:
            for addr in entry[0].buffer_addrs:
                reg.pop(addr, None)

    def for_rank(self, rank: int) -> "EmulatedSymmetricMemory":
        """The handle another emulated rank would hold for the same allocation."""
        assert 0 <= rank < self.world_size
        return EmulatedSymmetricMemory(self._group, rank)

    # ---- views
    def _view(self, rank, sizes, strides, dtype, storage_offset):
        itemsize = torch.empty((), dtype=dtype).element_size()
        g = self._group
        flat = g.slab[rank * g.buffer_stride:rank * g.buffer_stride + g.buffer_size].view(dtype)
        need = storage_offset + (1 + sum((n - 1) * s for n, s in zip(sizes, strides))
                                 if all(n > 0 for n in sizes) else 0)
        assert need * itemsize <= g.buffer_size, "view exceeds the symmetric buffer"
        # as_strided offsets are absolute within the storage, not relative to `flat`
        return flat.as_strided(tuple(sizes), tuple(strides), flat.storage_offset() + storage_offset)

    def get_buffer(self, rank: int, sizes: Sequence[int], dtype: torch.dtype,
                   storage_offset: int = 0) -> torch.Tensor:
        """Contiguous view of ``rank``'s buffer, ``storage_offset`` in elements
        (triton_all_gather_matmul.py:46-48)."""
        sizes = tuple(int(s) for s in sizes)
        strides = []
        acc = 1
        for n in reversed(sizes):
            strides.append(acc)
            acc *= max(n, 1)
        return self._view(int(rank), sizes, tuple(reversed(strides)), dtype, int(storage_offset))

    def all_buffers(self, sizes: Sequence[int], dtype: torch.dtype) -> torch.Tensor:
        """``[world_size, *sizes]`` view over every rank's buffer (no copy; an
        emulation-only convenience: on real peers these are eight allocations)."""
        sizes = tuple(int(s) for s in sizes)
        first = self.get_buffer(0, sizes, dtype)
        itemsize = first.element_size()
        g = self._group
        assert g.buffer_stride % itemsize == 0
        return g.slab.view(dtype).as_strided((self.world_size,) + sizes,
                                            (g.buffer_stride // itemsize,) + tuple(first.stride()),
                                            g.slab.view(dtype).storage_offset())

    def get_signal_pad(self, rank: int, sizes: Optional[Sequence[int]] = None,
                       dtype: torch.dtype = torch.int32) -> torch.Tensor:
        g = self._group
        pad = g.pads[rank * SIGNAL_PAD_SIZE:(rank + 1) * SIGNAL_PAD_SIZE].view(dtype)
        if sizes is not None:
            pad = pad[: math.prod(sizes)].view(*sizes)
        return pad

    # ---- status words written by kernels whose bounded spins expired
    @property
    def status(self) -> torch.Tensor:
        return self._group.status

    def check_status(self, reset: bool = True) -> None:
        """Synchronises and raises if a kernel reported a timed-out spin."""
        torch.cuda.synchronize(self.device)
        st = self._group.status.cpu().tolist()
        if reset:
            self._group.status.zero_()
        if st[0] != 0:
            text = _lib.STATUS_TEXT.get(st[0], f"status code {st[0]}")
            raise _lib.SmrError(f"{text}; waiter identity {st[1:]}")

    # ---- synchronisation
    def barrier(self, channel: int = 0) -> None:
        """Cross-rank barrier of the emulated group.  All emulated ranks issue
        their work from this one process onto the same stream, so stream order
        already gives what the cross-GPU barrier gives the reference
        (triton_all_gather_matmul.py:56,250); nothing is launched."""
        return None

    def stream_write_value32(self, addr: int, value: int) -> None:
        """Stream-ordered 32-bit flag write with release semantics
        (triton_all_gather_matmul.py:50-55)."""
        lib = _lib.load()
        stream = torch.cuda.current_stream(self.device).cuda_stream
        _lib.check(lib.smr_stream_write_value32(int(addr), int(value) & 0xFFFFFFFF, stream),
                   "stream_write_value32")


#: drop-in name used by the reference's modules
_SymmetricMemory = EmulatedSymmetricMemory

_backend_streams: Dict[int, "torch.cuda.Stream"] = {}


def _get_backend_stream() -> "torch.cuda.Stream":
    """Process-wide side stream for producer work, default priority
    (counterpart of torch.distributed._symmetric_memory._get_backend_stream,
    used at triton_all_gather_matmul.py:251-253,318)."""
    dev = torch.cuda.current_device()
    if dev not in _backend_streams:
        _backend_streams[dev] = torch.cuda.Stream(device=dev)
    return _backend_streams[dev]


def enable_symm_mem_for_group(group_name: str) -> None:
    """No-op: the emulated group needs no rendezvous."""
    return None
