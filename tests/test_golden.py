"""The committed golden vectors (tests/golden/*.npz, written by
tests/golden/make_vectors.py) against the oracle, and the C model of the barrier
protocol.  No GPU."""
import os
import subprocess

import numpy as np
import pytest

from oracle import oracle as O

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _load(name):
    return np.load(os.path.join(GOLDEN, name), allow_pickle=False)


def test_reduce_vectors():
    g = _load("reduce.npz")
    bufs = list(g["bf16_in"])
    assert np.array_equal(O.reduce_ref(bufs, "bf16"), g["bf16_out"])
    assert np.array_equal(O.reduce_ref_bf16_acc(bufs), g["bf16_out_bf16_acc"])
    assert np.array_equal(O.reduce_ref(list(g["fp32_in"]), "fp32").view(np.uint32), g["fp32_out"].view(np.uint32))
    # the inputs are the seeded generator's: N(0,1) per rank, seed = rank
    for r in range(8):
        assert np.array_equal(O.seeded_normal_bf16_bits(256, seed=r), g["bf16_in"][r])
    # fp32 accumulation and per-step bf16 rounding differ somewhere on real data
    assert not np.array_equal(g["bf16_out"], g["bf16_out_bf16_acc"])


def test_matmul_gemv_vectors():
    g = _load("ag_matmul.npz")
    assert np.array_equal(O.ag_matmul_ref(list(g["shards"]), g["b_nk"]), g["c"])
    v = _load("gemv.npz")
    out, partials = O.gemv_allreduce_ref(v["x"], v["w"], 8, return_partials=True)
    assert np.array_equal(out, v["out"]) and np.array_equal(partials.view(np.uint32), v["partials"].view(np.uint32))


def test_schedule_and_signal_vectors():
    g = _load("ref_schedule.npz")
    sched = O.ref_tile_schedule(1024, 256, 128, 128, 1, 128, 1, 8, 5)
    rows = [(p, t["pid_m"], t["pid_n"], t["comm_block"], int(t["local"]), t["a_row"])
            for p in sorted(sched) for t in sched[p]]
    assert np.array_equal(np.array(rows, dtype=np.int32), g["rows"])
    s = _load("signals.npz")
    assert O.all_gather_order(3, 8) == s["order_rank3"].tolist()
    assert O.all_gather_order(1, 4, 2) == s["order_rank1_ws4_splits2"].tolist()
    assert np.array_equal(O.signal_round_ref(s["round_src"], 5), s["round5"])


@pytest.mark.parametrize("ws,blocks,rounds", [(8, 4, 2000), (3, 2, 20000), (2, 1, 50000)])
def test_barrier_model_c(ws, blocks, rounds):
    """C11-atomics model of the CAS handshake (oracle/barrier_model.c): terminates,
    hands the payload over without stale reads, leaves every pad zero."""
    exe = os.path.join(ROOT, "oracle", "barrier_model")
    if not os.path.exists(exe):
        subprocess.run(["make", "-C", os.path.join(ROOT, "oracle")], check=True, capture_output=True)
    r = subprocess.run([exe, str(ws), str(blocks), str(rounds)], capture_output=True, text=True, timeout=60)
    assert r.returncode == 0, r.stdout + r.stderr
    assert "stale_reads=0 nonzero_slots=0" in r.stdout
