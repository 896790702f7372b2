"""The benchmark's contract: one GPU only, one JSON line with the agreed keys, figures that follow from each other,
and constants that point at files that exist."""
import json
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BENCH = os.path.join(ROOT, "bench.py")


def test_more_than_one_gpu_is_refused_with_a_message():
    r = subprocess.run([sys.executable, BENCH, "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert r.returncode == 2
    assert "one GPU" in r.stderr and r.stdout.strip() == ""


def test_traffic_constants_name_committed_profiles():
    sys.path.insert(0, ROOT)
    import bench
    assert bench.MEASURED_TRAFFIC
    for name, (nbytes, source) in bench.MEASURED_TRAFFIC.items():
        assert nbytes > 0 and source.startswith("profiles/"), name
        assert os.path.isfile(os.path.join(ROOT, source)), source


def test_headline_workload_is_the_baselines_and_its_bytes_are_the_documented_ones(pkg):
    wl = __import__("openvino_genai_amd.workloads", fromlist=["x"])
    spec = wl.make_spec(2)
    assert (spec["B"], spec["Hq"], spec["Hkv"], spec["D"], spec["bs"], spec["kv_dtype"]) == (64, 32, 8, 128, 32, "u8")
    assert int(spec["past_lens"].min()) == int(spec["past_lens"].max()) == 4096
    b = wl.algorithmic_bytes(spec, True)
    # 64 sequences x 4097 positions x 8 kv heads x 2 tensors x 136-byte rows, + Q, output, step arrays, scores
    assert b["kv"] == 64 * 4097 * 8 * 2 * 136 == 570564608
    assert b["total"] == b["kv"] + b["q_out"] + b["ints"] + b["scores"] == 572695816


@pytest.mark.gpu
def test_default_style_run_prints_one_json_line_with_the_contracts_keys():
    r = subprocess.run([sys.executable, BENCH, "--steps", "5", "--warmup", "2", "--settle-steps", "50", "--cpu-seconds", "1"],
                       capture_output=True, text=True, timeout=600, cwd=ROOT)
    assert r.returncode == 0, r.stderr[-2000:]
    lines = [ln for ln in r.stdout.splitlines() if ln.strip()]
    assert len(lines) == 1
    j = json.loads(lines[0])
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                "vs_baseline", "dtype", "data", "config", "roofline", "cpu_baseline"):
        assert key in j, key
    assert j["n_gpus"] == 1 and j["steps"] == 5 and j["warmup"] == 2 and j["higher_is_better"] is True
    assert j["vs_baseline"] is None and j["data"] == "synthetic" and j["unit"] == "GB/s"
    assert j["config"]["workload"] == "llama3_8b_decode_u8_b64_ctx4096" and "model" not in j["config"]
    # value = algorithmic bytes / step time
    assert j["value"] == pytest.approx(j["algorithmic_bytes"]["total"] / (j["ms_per_step"] * 1e-3) / 1e9, rel=1e-3)
    rf = j["roofline"]
    assert rf["bound"] == "hbm" and rf["peak"] == 8000.0 and rf["unit"] == "GB/s"
    assert rf["frac"] == pytest.approx(rf["achieved"] / rf["peak"], abs=2e-4)
    assert rf["achieved"] == pytest.approx(j["algorithmic_bytes"]["total"] / (rf["ms"] * 1e-3) / 1e9, rel=1e-3)
    assert 0.3 < rf["frac"] < 1.0 and rf["ms"] <= 1.05 * j["ms_per_step"]   # the kernel is part of the step, below the peak
    assert rf["traffic"] is None or rf["traffic"] >= 0.98 * j["algorithmic_bytes"]["total"]
    cb = j["cpu_baseline"]
    assert cb["kind"] == "port" and cb["unit"] == "GB/s" and cb["cores"] >= 1 and cb["value"] > 0 and cb["sample"]
    assert j["value"] > 50 * cb["value"]   # sanity, not a target: the GPU leg is not the checker in disguise
    # the child's device memory goes back to the driver shortly after it is reaped; tests that watch the free memory
    # (the allocation check of the static entry point) should not see that happen
    import time
    time.sleep(3)
