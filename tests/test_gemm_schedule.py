"""Host-only properties of the GEMM's tile order (the library's counterpart of the
index arithmetic at symm_mem_recipes/triton_all_gather_matmul.py:125-174): every
output tile exactly once, local comm block first, comm blocks in ring order, local
tiles never wait, one XCD's tiles of a pass form a compact patch."""
import collections

import pytest

from symm_mem_recipes import gemm_schedule


def _by_wg(s):
    by = collections.defaultdict(list)
    for t in s:
        by[t["wg"]].append(t)
    return by


def _covers_exactly(s, M, N):
    """The tiles are disjoint rectangles whose union is the whole output."""
    cells = set()
    for t in s:
        assert t["row0"] % 128 == 0 and t["col0"] % 32 == 0
        for r in range(t["row0"], t["row0"] + t["rows"], 128):
            for c in range(t["col0"], min(t["col0"] + t["cols"], (N + 31) // 32 * 32), 32):
                assert (r, c) not in cells, "tile overlap"
                cells.add((r, c))
    assert len(cells) == (M // 128) * ((N + 31) // 32)


@pytest.mark.parametrize("rank", [0, 3, 7])
@pytest.mark.parametrize("gated", [0, 2], ids=["ungated", "gated-whole-gpu"])
def test_schedule_config5_whole_gpu(lib, rank, gated):
    """A launch that has every compute unit (ungated, or gated by somebody who needs none):
    256x224 tiles, 64 x 16 = 1024 of them = 4 whole passes of 256 workgroups, where 256x256
    tiles are 896 = 4 passes of 224."""
    M, N, K, ws = 16384, 3584, 8192, 8
    assert lib.smr_ag_matmul_grid(M, N, K, ws, M // ws, gated) == 256
    s = gemm_schedule(M, N, K, rank, ws, M // ws, gated=gated)
    assert len(s) == 64 * 16
    assert {(t["rows"], t["cols"]) for t in s} == {(256, 224)}
    _covers_exactly(s, M, N)
    for t in s:
        assert t["comm_block"] == t["row0"] // 2048
        assert t["local"] == int(t["comm_block"] == rank)                  # only local tiles skip the wait
    by = _by_wg(s)
    assert len(by) == 256 and all(len(v) == 4 for v in by.values())
    for wg, tiles in by.items():
        assert [t["step"] for t in tiles] == list(range(len(tiles)))
        ring = [(t["comm_block"] - rank) % ws for t in tiles]
        assert ring == sorted(ring)                                        # ready order of the gather
    first = [t for t in s if t["step"] == 0]
    assert sum(t["local"] for t in first) == 8 * 16
    # XCD locality: the 32 tiles an XCD holds in the first pass share few A/B slabs
    for x in range(8):
        mine = [t for t in first if t["wg"] % 8 == x]
        assert len(mine) == 32
        slabs = len({t["row0"] for t in mine}) + len({t["col0"] for t in mine})
        assert slabs <= 20                                                 # 64 when unrelated


def test_schedule_config5_on_the_gated_grid(lib):
    """The same problem held to the gated launch's 224 workgroups (the grid limit): 256x256 tiles."""
    M, N, K, ws = 16384, 3584, 8192, 8
    try:
        assert lib.smr_set_ag_matmul_grid_limit(224) == 0
        s = gemm_schedule(M, N, K, 0, ws, M // ws, gated=0)
    finally:
        lib.smr_set_ag_matmul_grid_limit(0)
    assert len(s) == 64 * 14 and {(t["rows"], t["cols"]) for t in s} == {(256, 256)}
    assert len(_by_wg(s)) == 224


@pytest.mark.parametrize("rank", [0, 3, 7])
def test_schedule_config5_gated(rank):
    """Gated: the same full tiles in the same ready order on a grid that leaves the
    producer its compute units; only tiles of the local comm block skip the wait."""
    M, N, K, ws = 16384, 3584, 8192, 8
    s = gemm_schedule(M, N, K, rank, ws, M // ws, gated=True)
    _covers_exactly(s, M, N)
    by = _by_wg(s)
    assert len(by) == 224
    for wg, tiles in by.items():
        assert [t["cols"] for t in tiles] == [256, 256, 256, 256]
        ring = [(t["comm_block"] - rank) % ws for t in tiles]
        assert ring == sorted(ring)
    for t in s:
        assert t["comm_block"] == t["row0"] // 2048
        assert t["local"] == int(t["comm_block"] == rank)
    # a pass needs two comm blocks: the local one and the first to arrive, then the next two
    for step in range(4):
        assert {(t["comm_block"] - rank) % ws for t in s if t["step"] == step} == {2 * step, 2 * step + 1}


@pytest.mark.parametrize("M,N,K,ws,splits", [(1024, 256, 256, 8, 1), (2048, 384, 512, 8, 1),
                                             (2048, 264, 128, 4, 2), (512, 128, 64, 2, 2),
                                             (4096, 1792, 4096, 8, 1)])
def test_schedule_other_shapes(M, N, K, ws, splits):
    comm = M // ws // splits
    for rank in range(ws):
        s = gemm_schedule(M, N, K, rank, ws, comm)
        assert comm % s[0]["rows"] == 0
        _covers_exactly(s, M, N)
        for t in s:
            owner = t["comm_block"] // splits
            assert t["local"] == int(owner == rank)
        for tiles in _by_wg(s).values():
            first_local = rank * splits
            ring = [(t["comm_block"] - first_local) % (ws * splits) for t in tiles]
            assert ring == sorted(ring)


def test_grid_leaves_room_for_the_producer(lib):
    # gated launches never take every compute unit (256 assumed without a GPU)
    for (M, N, K) in [(16384, 3584, 8192), (16384, 6656, 16384), (4096, 1792, 4096), (32768, 8192, 1024)]:
        gated = lib.smr_ag_matmul_grid(M, N, K, 8, M // 8, 1)
        ungated = lib.smr_ag_matmul_grid(M, N, K, 8, M // 8, 0)
        assert 8 <= gated <= 248 and gated % 8 == 0
        assert gated <= ungated <= 256


def test_fused_plan_splits_the_gpu(lib):
    """smr_ag_matmul_plan: GEMM grid + producer fit the GPU (256 compute units assumed
    without one) and the grid is the one the gated GEMM launches; both forms come with an
    estimate, and a problem too small to hide the copy behind is planned as copy-then-multiply."""
    import ctypes
    plans = {}
    for (M, N, K) in [(16384, 3584, 8192), (16384, 6656, 16384), (8192, 3584, 8192), (16384, 1792, 4096),
                      (4096, 8192, 8192), (2048, 4096, 2048), (1024, 256, 256), (8192, 1792, 4096),
                      (4096, 3584, 8192)]:
        out = (ctypes.c_int32 * 5)()
        assert lib.smr_ag_matmul_plan(M, N, K, 8, M // 8, out) == 0
        grid, wgs, fused_us, sequential_us, sequential = list(out)
        assert grid % 8 == 0 and 8 <= grid <= 248
        assert grid == lib.smr_ag_matmul_grid(M, N, K, 8, M // 8, 1)
        assert 1 <= wgs <= 128 and grid + wgs <= 256
        assert fused_us > 0 and sequential_us > 0
        assert sequential == (1 if sequential_us < 0.98 * fused_us else 0)
        plans[(M, N, K)] = (grid, wgs, sequential)
    # (the choices below are the ones launches timed on MI355X bear out)
    assert plans[(16384, 3584, 8192)] == (224, 32, 0)
    assert plans[(16384, 6656, 16384)][2] == 0
    assert plans[(4096, 8192, 8192)][2] == 1 and plans[(2048, 4096, 2048)][2] == 1
    assert plans[(8192, 1792, 4096)][2] == 1 and plans[(4096, 3584, 8192)][2] == 1
    assert plans[(8192, 3584, 8192)][2] == 0 and plans[(16384, 1792, 4096)][2] == 1
    # a problem with few passes leaves the copy more of the GPU
    assert plans[(2048, 4096, 2048)][1] > plans[(16384, 3584, 8192)][1]
    out = (ctypes.c_int32 * 5)()
    assert lib.smr_ag_matmul_plan_fp8(16384, 3584, 8192, 8, 2048, out) == 0
    assert list(out)[:2] == [224, 32] and out[4] == 0
    # (e4m3fn: the narrow problem is the faster one copied first, 124 against 139 us)
    assert lib.smr_ag_matmul_plan_fp8(16384, 1792, 4096, 8, 2048, out) == 0 and out[4] == 1
    assert lib.smr_ag_matmul_plan_fp8(8192, 3584, 8192, 8, 1024, out) == 0 and out[4] == 0
    assert lib.smr_ag_matmul_plan_fp8(16384, 3584, 8192 + 64, 8, 2048, out) == -2      # K % 128
    assert lib.smr_ag_matmul_plan(1000, 256, 256, 8, 125, out) == -2                   # unsupported shape
    assert lib.smr_ag_matmul_plan(1024, 256, 256, 8, 128, None) == -1


def test_timetable_of_a_gated_launch(lib):
    """smr_ag_matmul_pace, the timetable smr_all_gather_beside is given: a world_size-th of an estimate that is
    within a fifth of what the ungated launches take on MI355X (256 compute units assumed without a GPU), the
    ranks of the first pass, nothing to spread for a single pass, and the GEMM's own refusals."""
    import ctypes
    out = (ctypes.c_int32 * 2)()
    measured = {(16384, 3584, 8192): (630, 2), (16384, 1792, 4096): (178, 4), (16384, 7168, 8192): (1250, 2),
                (8192, 3584, 8192): (323, 4), (16384, 8192, 2048): (406, 1)}
    for (M, N, K), (us, lead) in measured.items():
        assert lib.smr_ag_matmul_pace(M, N, K, 8, M // 8, 2, out) == 0
        assert 0.8 * us <= 8 * out[0] <= 1.2 * us, (M, N, K, list(out), us)
        assert out[1] == lead, (M, N, K, list(out))
    assert lib.smr_ag_matmul_pace(4096, 3584, 8192, 8, 512, 2, out) == 0 and list(out) == [0, 8]     # one pass
    assert lib.smr_ag_matmul_pace(16384, 3584, 8192, 8, 2048, 1, out) == 0
    assert 0.4 * 630 <= 8 * out[0] <= 0.65 * 630
    assert lib.smr_ag_matmul_pace(1000, 256, 256, 8, 125, 2, out) == -2
    assert lib.smr_ag_matmul_pace(16384, 3584, 8192 + 64, 8, 2048, 1, out) == -2
    assert lib.smr_ag_matmul_pace(1024, 256, 256, 8, 128, 4, out) == -1
    assert lib.smr_ag_matmul_pace(1024, 256, 256, 8, 128, 2, None) == -1


def test_schedule_rejects_bad_shapes():
    with pytest.raises(AssertionError):
        gemm_schedule(1000, 256, 256, 0, 8, 125)        # rows per flag not a multiple of 128
    with pytest.raises(AssertionError):
        gemm_schedule(1024, 256, 100, 0, 8, 128)        # K not a multiple of 64
    with pytest.raises(AssertionError):
        gemm_schedule(1024, 252, 256, 0, 8, 128)        # N not a multiple of 8
    with pytest.raises(AssertionError):
        gemm_schedule(1024, 256, 256, 8, 8, 128)        # rank out of range


def _row_swizzle_from_source():
    """The kernel's row_swizzle, taken from the source text (the expression is valid Python)."""
    import os
    import re
    src = open(os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))),
                            "symm-mem-recipes_amd", "csrc", "ag_matmul.hip")).read()
    m = re.search(r"inline int row_swizzle\(int r\) \{\s*return (.*?);\s*\}", src, re.S)
    assert m, "row_swizzle not found"
    expr = m.group(1)
    return lambda r: eval(expr, {"r": r})


def _lds_columns(accesses):
    """16-byte columns of the 256-byte bank row that a set of (row, position) accesses to a slab
    touches: a slab row is 128 bytes, so even rows lie in columns 0-7 and odd rows in 8-15."""
    return [(row & 1) * 8 + pos for row, pos in accesses]


def test_fragment_reads_are_free_of_bank_conflicts():
    """A 128-bit LDS read is served 16 lanes at a time (lanes 8g..8g+7 with 32+8g..32+8g+7), and
    those 16 must fall into 16 different 16-byte columns.  Checked for the bf16 fragments
    (lane l: row l & 15, chunk 4 * kk + (l >> 4)), the e4m3fn fragments (row l & 15, chunks
    2 * (l >> 4) + q) and for every 16-row fragment of a slab, with the swizzle the kernel uses."""
    sw = _row_swizzle_from_source()
    groups = [[8 * g + i for i in range(8)] + [32 + 8 * g + i for i in range(8)] for g in range(4)]
    for frag_row0 in range(0, 256, 16):
        for lanes in groups:
            for kk in range(2):                    # bf16: K step kk of a slab
                acc = [(frag_row0 + (l & 15), (4 * kk + (l >> 4)) ^ sw((frag_row0 + (l & 15)) & 15)) for l in lanes]
                assert len(set(_lds_columns(acc))) == 16, ("bf16", frag_row0, lanes, kk)
            for q in range(2):                     # e4m3fn: first and second half of the lane's 32 bytes
                acc = [(frag_row0 + (l & 15), (2 * (l >> 4) + q) ^ sw((frag_row0 + (l & 15)) & 15)) for l in lanes]
                assert len(set(_lds_columns(acc))) == 16, ("e4m3fn", frag_row0, lanes, q)


def test_tile_loads_fill_every_chunk_of_a_slab_once():
    """A direct-to-LDS load lands lane l of load group q at byte q * 1024 + l * 16, i.e. row
    q * 8 + (l >> 3), position l & 7; the lane fetches chunk (l & 7) ^ swizzle(l >> 3) ^ ((q & 1) << 2)
    of that row.  Position p of row r must hold chunk p ^ row_swizzle(r): every chunk of every row
    exactly once."""
    sw = _row_swizzle_from_source()
    for q in range(32):
        for l in range(64):
            row, pos = q * 8 + (l >> 3), l & 7
            chunk = ((l & 7) ^ sw(l >> 3)) ^ ((q & 1) << 2)
            assert chunk == pos ^ sw(row & 15), (q, l)
