#!/usr/bin/env python3
"""Writes the small golden vectors under tests/golden/ from the CPU oracle.

The reference holds no fixture files and cannot be executed here, so these
vectors do not come from it: they freeze the oracle's outputs (which
tests/test_oracle.py pins against exact arithmetic and library routines) so that a
later change to the oracle, or to the seeded input generators, cannot go unnoticed,
and they give the GPU tests a target that does not depend on the oracle's code.

    python tests/golden/make_vectors.py        # rewrites tests/golden/*.npz
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
from oracle import oracle as O  # noqa: E402


def main():
    # one-shot all-reduce: 8 ranks x 256 elements, bf16 and fp32, N(0,1) seeded per rank
    bufs = [O.seeded_normal_bf16_bits(256, seed=r) for r in range(8)]
    f32 = [O.seeded_normal_f32(256, seed=r) for r in range(8)]
    np.savez(os.path.join(HERE, "reduce.npz"),
             bf16_in=np.stack(bufs), bf16_out=O.reduce_ref(bufs, "bf16"),
             bf16_out_bf16_acc=O.reduce_ref_bf16_acc(bufs),
             fp32_in=np.stack(f32), fp32_out=O.reduce_ref(f32, "fp32"))
    # all-gather matmul: 4 shards of [128, 64], B [72, 64] (ragged column tile)
    shards = [O.seeded_normal_bf16_bits(128 * 64, seed=r, std=0.02).reshape(128, 64) for r in range(4)]
    b = O.seeded_normal_bf16_bits(72 * 64, seed=100, std=0.02).reshape(72, 64)
    np.savez(os.path.join(HERE, "ag_matmul.npz"), shards=np.stack(shards), b_nk=b,
             c=O.ag_matmul_ref(shards, b))
    # split-K GEMV: x [4, 256], W [256, 128], 8 K-shards
    x = O.seeded_normal_bf16_bits(4 * 256, seed=0).reshape(4, 256)
    w = O.seeded_normal_bf16_bits(256 * 128, seed=1, std=0.02).reshape(256, 128)
    out, partials = O.gemv_allreduce_ref(x, w, 8, return_partials=True)
    np.savez(os.path.join(HERE, "gemv.npz"), x=x, w=w, out=out, partials=partials)
    # reference tile schedule of a toy shape (M=1024 N=256, 128x128 tiles, group 2, rank 1, 8 ranks, 5 programs)
    sched = O.ref_tile_schedule(1024, 256, 128, 128, 1, 128, 1, 8, 5)
    rows = [(p, t["pid_m"], t["pid_n"], t["comm_block"], int(t["local"]), t["a_row"])
            for p in sorted(sched) for t in sched[p]]
    np.savez(os.path.join(HERE, "ref_schedule.npz"), rows=np.array(rows, dtype=np.int32))
    # producer order and a signal round checksum
    src = (np.arange(2 * 3 * 8, dtype=np.uint32) * np.uint32(2654435761)).reshape(2, 3, 8)
    np.savez(os.path.join(HERE, "signals.npz"), order_rank3=np.array(O.all_gather_order(3, 8), np.int32),
             order_rank1_ws4_splits2=np.array(O.all_gather_order(1, 4, 2), np.int32),
             round_src=src, round5=O.signal_round_ref(src, 5))


if __name__ == "__main__":
    main()
