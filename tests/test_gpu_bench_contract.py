"""The bench line keeps its contract: one JSON object on stdout with the driver's fields, the roofline and (when asked
for) the CPU baseline; more than one GPU is refused with a message."""
import json
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.mark.gpu
def test_bench_line_fields():
    out = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "1", "--steps", "2", "--warmup", "1",
                          "--skip-sub", "--skip-cpu"], capture_output=True, text=True, timeout=300, cwd=ROOT)
    assert out.returncode == 0, out.stderr[-2000:]
    lines = [l for l in out.stdout.strip().splitlines() if l.startswith("{")]
    assert len(lines) == 1
    b = json.loads(lines[0])
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                "vs_baseline", "dtype", "data", "config", "roofline"):
        assert key in b, key
    assert b["n_gpus"] == 1 and b["steps"] == 2 and b["warmup"] == 1 and b["higher_is_better"] is True
    assert b["unit"] == "TOPS" and b["dtype"] == "int8" and b["data"] == "synthetic" and b["vs_baseline"] is None
    assert "workload" in b["config"] and "model" not in b["config"]
    r = b["roofline"]
    assert r["bound"] == "mfma" and r["unit"] == "TOP/s" and r["peak"] == 5000.0
    assert abs(r["frac"] - r["achieved"] / r["peak"]) < 1e-3
    assert 0.05 < r["frac"] < 1.0 and b["value"] > 100.0
    # value is ops per step over the step time, and the step time is the declared method's (graph replay)
    assert abs(b["value"] - b["config"]["ops_per_step"] / (b["ms_per_step"] * 1e-3) / 1e12) < 0.01 * b["value"]
    assert b["ms_per_step"] == b["config"]["ms_per_step_graph"] and "ms_per_step_eager" in b["config"]
    # the HBM traffic figure says where it comes from: a separate counter run, not this one
    assert r["traffic"] is None or "profiles/" in r["traffic_source"]
    # the matrix-pipe probe's figure rides along as context: below the published peak, above what the GEMMs reach
    m = r["sustained_mfma_measured"]
    assert m is not None and 0 < m["tops"] <= r["peak"] and 0 < m["zeros_no_reads_tops"] <= r["peak"]
    assert abs(m["frac_of_it"] - r["achieved"] / m["tops"]) < 1e-3


@pytest.mark.gpu
def test_probe_and_timeline_modes_print_one_json_line_each():
    """The two measurement modes behind profiles/mfma_power_limited_peak.md and the GEMM timeline profiles: structure
    only (one JSON line, the expected keys, parts that add up to the whole); what the figures are is the profiles'
    business, since a throttled clock moves every one of them."""
    out = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--mfma-probe"], capture_output=True, text=True,
                         timeout=300, cwd=ROOT)
    assert out.returncode == 0, out.stderr[-2000:]
    lines = [l for l in out.stdout.strip().splitlines() if l.startswith("{")]
    assert len(lines) == 1
    runs = json.loads(lines[0])["mfma_power_limited_peak"]["runs"]
    assert len(runs) == 8 and all(r["tops"] > 0 and r["clock_ticks_per_mfma"] > 0 for r in runs)
    assert [r["waves_per_simd"] for r in runs] == [1, 2] * 4
    out = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gemm-timeline"], capture_output=True,
                         text=True, timeout=400, cwd=ROOT)
    assert out.returncode == 0, out.stderr[-2000:]
    lines = [l for l in out.stdout.strip().splitlines() if l.startswith("{")]
    assert len(lines) == 1
    tl = json.loads(lines[0])["gemm_timeline"]
    for name in ("qkv", "down"):
        t = tl[name]["ticks"]
        parts = t["prologue"] + t["stage_loop"] + min(t["exchange_and_stores_issued"]) + t["stores_acknowledged"]
        assert 0.9 * parts <= t["whole_kernel"] <= 1.1 * (parts + 3000)
        assert tl[name]["workgroups"] > 0 and tl[name]["stages"] in (32, 112) and tl[name]["kernel_us_event"] > 0
    b = tl["batch"]
    # every tile of the four projections left its three clock reads: 8 row tiles x (24 + 56 + 56 + 16) column tiles
    assert b["tiles"] == 8 * (24 + 56 + 56 + 16) and 0 < b["workgroups"] <= 512
    assert set(b["per_tile_depth"]) == {"stages_32", "stages_112"}
    assert sum(v["tiles"] for v in b["per_tile_depth"].values()) == b["tiles"]
    assert b["loop_ticks_all_tiles"] > 0 and b["convert_and_store_ticks_all_tiles"] > 0
    # what the workgroups spent inside tiles cannot exceed workgroups x the launch's span (ticks at the measured clock)
    span_ticks = b["first_tile_start_to_last_store_us"] * b["clock_mhz"]
    assert b["loop_ticks_all_tiles"] + b["convert_and_store_ticks_all_tiles"] <= 1.05 * b["workgroups"] * span_ticks


def test_cpu_baseline_leg_pins_its_threads_per_numa_node():
    """The CPU leg without a GPU: node CPU lists come from sysfs and lie inside the process's affinity mask, every
    OpenMP thread gets pinned, and the record carries a figure for every config."""
    sys.path.insert(0, ROOT)
    sys.path.insert(0, os.path.join(ROOT, "mojo-linuxperiments_amd"))
    sys.path.insert(0, os.path.join(ROOT, "oracle"))
    import bench
    import cpu_oracle as orc
    nodes = bench.node_cpu_lists()
    allowed = os.sched_getaffinity(0)
    assert nodes and all(cpus and set(cpus) <= allowed for cpus in nodes.values())
    assert sum(len(c) for c in nodes.values()) <= len(allowed)
    first = sorted(nodes)[0]
    try:
        assert orc.pin_threads(nodes[first][:1] * orc.num_threads()) == orc.num_threads()
    finally:
        # give the team its CPUs back for the tests that follow
        every = sorted(allowed)
        orc.pin_threads([every[i % len(every)] for i in range(orc.num_threads())])
    src = open(os.path.join(ROOT, "bench.py")).read()
    for key in ("cfg0_linear_m32", "cfg1_decode_gemv", "cfg2_decode_attention", "cfg4_moe_layer", "per_config",
                "threads_pinned"):
        assert '"%s"' % key in src[src.index("def cpu_baseline"):], key


def test_bench_refuses_more_than_one_gpu():
    out = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True,
                         timeout=120, cwd=ROOT)
    assert out.returncode != 0
    assert "ONE GPU" in (out.stderr + out.stdout)
