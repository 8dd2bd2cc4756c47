"""Host-side contract of bench.py that needs no GPU: one GPU only, and the hardware-counter
figures it prints come from the file kept beside the profiler summaries."""
import json
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_more_than_one_gpu_is_refused():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"],
                       capture_output=True, text=True, timeout=120)
    assert r.returncode != 0
    assert "--gpus must be 1" in r.stderr
    assert r.stdout.strip() == ""                     # no JSON line for a run that did not happen


def test_counter_figures_name_their_summaries():
    sys.path.insert(0, ROOT)
    import bench
    c = bench._counters()
    with open(os.path.join(ROOT, "profiles", "counters.json")) as f:
        assert c == json.load(f)
    # every group points at the summary it was taken from, and that summary quotes the figure
    for group in ("reduce_traffic_bytes", "gemm", "gemm_fp8"):
        src = os.path.join(ROOT, c[group]["source"])
        assert os.path.isfile(src), src
    reduce_md = open(os.path.join(ROOT, c["reduce_traffic_bytes"]["source"])).read()
    assert f"{c['reduce_traffic_bytes']['64']:,}" in reduce_md
    gemm_md = open(os.path.join(ROOT, c["gemm"]["source"])).read()
    for form in ("fused", "ungated", "ungated_on_the_gated_grid", "hipblaslt"):
        entry = c["gemm"][form]
        assert 0.5 < entry["mfma_busy"] < 1.0 and entry["traffic"] > 4 * 10 ** 8
        assert f"**{entry['mfma_busy']:.3f}**" in gemm_md, form
    assert f"{c['gemm_fp8']['fused']['traffic']:,}" in gemm_md
