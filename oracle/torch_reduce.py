"""The one-shot all-reduce restated on torch-CPU tensors.  TEST INFRASTRUCTURE ONLY.

The same arithmetic as ``oracle.reduce_ref`` (fp32 accumulator that starts at +0, the
peers added one at a time in rank order 0..world_size-1, one rounding to the buffers'
dtype at the end; symm_mem_recipes/triton_one_shot_all_reduce.py:84-89 with the fp32
accumulator in place of the reference's per-step bf16 rounding, :36-49), written the
way a torch user would write the CPU path: ``acc += buf.float()`` per peer, then a
cast.  It exists so that the benchmark can time the CPU baseline with torch's own
threading, at all host cores and at one; tests pin it bit for bit against the numpy
oracle.  Imported only by tests and by the benchmark's CPU-baseline leg.
"""
from __future__ import annotations

from typing import Sequence

import torch


def reduce_ref_torch(bufs: Sequence[torch.Tensor]) -> torch.Tensor:
    """``bufs``: world_size CPU tensors of one shape, bfloat16 or float32."""
    acc = torch.zeros(bufs[0].shape, dtype=torch.float32)
    for b in bufs:
        acc += b.float()
    return acc.to(bufs[0].dtype)


def seeded_normal(numel: int, seed: int, dtype: torch.dtype = torch.bfloat16) -> torch.Tensor:
    """N(0, 1) values of a per-rank generator, generated in fp32 and cast."""
    g = torch.Generator()
    g.manual_seed(seed)
    return torch.randn(numel, generator=g, dtype=torch.float32).to(dtype)
