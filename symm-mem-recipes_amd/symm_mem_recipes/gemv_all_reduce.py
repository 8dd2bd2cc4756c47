"""Split-K GEMV fused with an all-reduce of the partial results through
signal-pad flags.  The reference has no counterpart module; the flag protocol is
the one of symm_mem_recipes/triton_barrier.py:119-129 and
symm_mem_recipes/triton_all_gather_matmul.py:72-95.

``W`` ([K, N], row-major) is split along K into ``world_size`` shards, one per
emulated rank (the kernel may cut a shard further into sub-shards to fill the
chip); every producer multiplies its share of ``x`` with its share of ``W`` in
fp32, publishes the partial and raises a flag; the partials are added in rank
order 0..world_size-1 in fp32 and rounded to bf16 once.
"""
from __future__ import annotations

from typing import Optional

import torch

from . import _lib


class GemvWorkspace:
    """Scratch the kernel needs: fp32 partials, the flag array (zero between
    calls) and status words."""

    def __init__(self, batch: int, N: int, world_size: int, device, K: int = 0):
        lib = _lib.load()
        self.batch, self.N, self.world_size = batch, N, world_size
        # partial producers per column block: the ranks, each possibly cut into K sub-shards
        self.senders = lib.smr_gemv_senders(N, K, world_size) if K else 8 * world_size
        self.partials = torch.empty(self.senders, batch, N, dtype=torch.float32, device=device)
        # per column block one flag per producer and one arrival word
        self.flags = torch.zeros(lib.smr_gemv_flag_blocks(N) * (self.senders + 1), dtype=torch.int32, device=device)
        self.status = torch.zeros(_lib.STATUS_WORDS, dtype=torch.int32, device=device)

    def check_status(self) -> None:
        torch.cuda.synchronize(self.status.device)
        st = self.status.cpu().tolist()
        self.status.zero_()
        if st[0] != 0:
            raise _lib.SmrError(f"{_lib.STATUS_TEXT.get(st[0], st[0])}; waiter identity {st[1:]}")


def gemv_all_reduce(x: torch.Tensor, w: torch.Tensor, world_size: int = 8,
                    workspace: Optional[GemvWorkspace] = None,
                    out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``x`` [batch, K] bf16 (batch <= 8), ``w`` [K, N] bf16 -> [batch, N] bf16."""
    assert x.dtype == torch.bfloat16 and w.dtype == torch.bfloat16, "Only bfloat16 is supported for now."
    assert x.dim() == 2 and w.dim() == 2 and x.shape[1] == w.shape[0]
    assert x.is_contiguous() and w.is_contiguous()
    batch, K = x.shape
    N = w.shape[1]
    assert 1 <= batch <= 8, "batch must be 1..8"
    assert K % world_size == 0, "K must split evenly over the ranks"
    if workspace is None:
        workspace = GemvWorkspace(batch, N, world_size, x.device, K)
    assert (workspace.batch, workspace.N, workspace.world_size) == (batch, N, world_size)
    lib = _lib.load()
    senders = lib.smr_gemv_senders(N, K, world_size)
    # (the launch shape is a process-wide knob: a workspace made under another setting may be too small)
    assert workspace.senders >= senders, "workspace was built for fewer partial producers"
    assert workspace.flags.numel() >= lib.smr_gemv_flag_words(N, K, world_size), "workspace has too few flags"
    if out is None:
        out = torch.empty(batch, N, dtype=torch.bfloat16, device=x.device)
    rc = lib.smr_gemv_allreduce(
        x.data_ptr(), w.data_ptr(), workspace.partials.data_ptr(), workspace.partials.numel() * 4,
        workspace.flags.data_ptr(), workspace.flags.numel(), out.data_ptr(), batch, K, N, world_size,
        workspace.status.data_ptr(), torch.cuda.current_stream(x.device).cuda_stream)
    _lib.check(rc, "gemv_all_reduce")
    return out
