"""bench.py keeps its output contract: one JSON line with the agreed keys, the roofline and
CPU-baseline objects, for the forward and the search workload (small shapes here)."""
import json
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
pytestmark = pytest.mark.gpu

KEYS = ["metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better",
        "scaling", "vs_baseline", "dtype", "data", "config"]


def run_bench(*args):
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py")] + list(args),
                       capture_output=True, text=True, timeout=600, cwd=ROOT)
    return r


def test_forward_line():
    print("case: bench forward 2x64 b8", flush=True)
    r = run_bench("--blocks", "2", "--filters", "64", "--batch", "8", "--steps", "3", "--warmup", "1",
                  "--profile-reps", "1")
    assert r.returncode == 0, r.stderr[-2000:]
    lines = [l for l in r.stdout.splitlines() if l.strip()]
    assert len(lines) == 1
    d = json.loads(lines[0])
    for k in KEYS:
        assert k in d, k
    assert d["n_gpus"] == 1 and d["steps"] == 3 and d["warmup"] == 1
    assert d["value"] > 0 and d["ms_per_step"] > 0 and d["vs_baseline"] is None
    assert "workload" in d["config"] and "model" not in d["config"]
    rf = d["roofline"]
    for k in ("bound", "achieved", "peak", "unit", "frac", "traffic"):
        assert k in rf, k
    assert rf["bound"] == "mfma" and rf["unit"] == "TFLOP/s" and 0 < rf["frac"] < 1
    assert abs(rf["frac"] - rf["achieved"] / rf["peak"]) < 1e-9
    # the same launch priced launch to launch (what a kernel trace reads): the same work over
    # another duration (the longer one at full size; on this test's tiny network the events'
    # own overhead can make theirs the longer)
    l2l = rf["launch_to_launch"]
    assert l2l["avg_launch_us"] > 0 and 0 < l2l["frac"] < 1
    assert abs(l2l["frac"] * l2l["avg_launch_us"] - rf["frac"] * rf["avg_launch_us"]) < 1e-6
    cb = d["cpu_baseline"]
    for k in ("value", "unit", "cores", "kind", "sample"):
        assert k in cb, k
    assert cb["kind"] == "port" and cb["value"] > 0 and cb["cores"] >= 1
    assert cb["raw_policy_plane_rel_l2_vs_gpu"] < 2e-2      # the spot check against the oracle
    for name in ("out_in_transform", "in_transform", "out_transform"):
        t = d["roofline_transforms"][name]
        assert t["bound"] == "hbm" and 0 < t["frac"] < 1
    # the figures beside the headline one: host buffers (PCIe inside the timed region), the
    # repeated blocks, the plain-copy floor, the same net in fp32 and the smaller configurations
    hb = d["host_buffers"]
    assert hb["value"] > 0 and "PCIe" in hb["note"] and d["config"]["inputs"].startswith("device")
    bk = d["blocks_of_k"]
    assert bk["blocks"] == 5 and bk["forwards_per_block"] == 200 and bk["min"] <= bk["median"] <= bk["max"]
    cf = d["hbm_copy_floor"]
    assert cf["us_per_launch"] > 0 and 0 < cf["frac_of_hbm_peak"] < 1.5
    assert d["fp32"]["value"] > 0 and 0 < d["fp32"]["gemm_frac_of_mfma_peak"] < 1
    assert set(d["configs"]) == {"6x128 fp32 b1", "15x192 fp32 b8", "20x256 fp16 b32"}
    for c in d["configs"].values():
        assert c["value"] > 0 and c["one_lane"] > 0
    assert d["configs"]["6x128 fp32 b1"]["cpu_oracle"]["value"] > 0
    lb = d["latency_by_batch"]
    assert 0 < lb["b1_ms"] <= lb["b32_ms"] and lb["b16_graph_replay_ms"] > 0


def test_more_than_one_gpu_is_refused():
    r = run_bench("--gpus", "2")
    assert r.returncode != 0
    assert "one GPU" in r.stderr and r.stdout.strip() == ""


def test_search_line():
    print("case: bench search 2x64", flush=True)
    r = run_bench("--workload", "search", "--blocks", "2", "--filters", "64", "--batch", "8",
                  "--threads", "12", "--visits", "100", "--moves", "4")
    assert r.returncode == 0, r.stderr[-2000:]
    d = json.loads(r.stdout.strip().splitlines()[-1])
    for k in KEYS:
        assert k in d, k
    assert d["unit"] == "visits/s" and d["value"] > 0
    assert 0 < d["batch_fill"] <= 1 and d["steps"] == 4 and len(d["moves"]) == 4
