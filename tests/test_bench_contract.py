"""bench.py's command-line contract: one JSON line with the agreed keys; more than one GPU is refused."""
import json
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_more_than_one_gpu_is_refused():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert r.returncode != 0 and "one GPU" in (r.stderr + r.stdout)


CONTRACT_KEYS = ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling", "vs_baseline",
                 "dtype", "data", "config", "roofline")
LINE_LIMIT = 6000  # characters of the one stdout line: what reads the line keeps a bounded tail of stdout


def test_final_line_of_a_full_run_is_short_and_keeps_the_contract():
    """The line bench.py prints is built by final_line() from the full result.  With every default leg in the result
    (tests/golden/bench_full_sample.json: a full default run of this bench on an MI355X) it stays a few KB and still
    carries the contract keys, the roofline and the CPU baseline; the per-row tables stay out of it."""
    sys.path.insert(0, ROOT)
    import bench

    full = json.load(open(os.path.join(ROOT, "tests", "golden", "bench_full_sample.json")))
    for leg in ("single_launch", "other_encodings", "configs", "density_sweep", "cpu_baseline", "layer_sequence", "launch_plans", "quantising_calls"):
        assert full.get(leg), leg
    assert len(json.dumps(full)) > 4 * LINE_LIMIT  # the sample really holds the tables
    line = bench.final_line(full)
    assert len(line) < LINE_LIMIT and "\n" not in line
    j = json.loads(line)
    for k in CONTRACT_KEYS + ("cpu_baseline", "targets", "summary", "single_launch_cold_us"):
        assert k in j, k
    for k in ("bound", "achieved", "peak", "unit", "frac", "traffic", "kernel", "launch_us"):
        assert k in j["roofline"], k
    for k in ("value", "unit", "cores", "kind", "sample"):
        assert k in j["cpu_baseline"], k
    assert "configs" not in j and "density_sweep" not in j
    for k in ("cfg1_m4", "cfg2_delta_fp16", "cfg3_layer_summed", "cfg4_large", "layer_sequence", "density_lists_over_i2s", "launch_plans_model_vs_tuned"):
        assert k in j["summary"], k


@pytest.mark.gpu
def test_json_line_has_the_contract_keys(tmp_path):
    detail = str(tmp_path / "detail.json")
    # every default leg, with short timing loops: the line that is checked is the line a default run prints
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--steps", "8", "--warmup", "2", "--no-cpu", "--reps", "48",
                        "--detail", detail], capture_output=True, text=True, timeout=900)
    assert r.returncode == 0, r.stderr[-2000:]
    lines = [l for l in r.stdout.splitlines() if l.strip()]
    assert len(lines) == 1 and len(lines[0]) < LINE_LIMIT
    j = json.loads(lines[0])
    for k in CONTRACT_KEYS:
        assert k in j, k
    full = json.load(open(detail))
    assert full["configs"]["cfg3_layer"]["shapes"] and full["density_sweep"]["shapes"] and full["layer_sequence"]["rows"] and full["launch_plans"]["rows"]
    assert "layer_sequence" in j["summary"] and "cfg4_large" in j["summary"]
    assert j["n_gpus"] == 1 and j["steps"] == 8 and j["warmup"] == 2 and j["higher_is_better"] is False and j["vs_baseline"] is None
    assert "workload" in j["config"] and "model" not in j["config"]
    rf = j["roofline"]
    assert rf["bound"] == "hbm" and rf["peak"] == 8000.0 and rf["unit"] == "GB/s"
    assert abs(rf["frac"] - rf["achieved"] / rf["peak"]) < 1e-3 and 0.3 < rf["frac"] < 1.0
    assert abs(j["value"] * 32 - rf["launch_us"]) < 0.05 * rf["launch_us"]
    assert 0.5 < rf["frac_of_streaming_read"] < 1.3
    side = json.load(open(os.path.join(ROOT, "profiles", "traffic_lists_kernel_batched_i8_u16_cfg0.json")))
    assert rf["traffic"] == side["traffic_bytes_per_launch"] and rf["traffic_measured_at_commit"] == side["measured_at_commit"]
    assert rf["algorithmic_bytes_per_launch"] == side["algorithmic_bytes_per_launch"]


def test_traffic_sidecar_is_consistent():
    """roofline.traffic comes from a counter run kept in profiles/: the file names its commit and commands, and its
    bytes follow from its own counter readings and scale factors."""
    side = json.load(open(os.path.join(ROOT, "profiles", "traffic_lists_kernel_batched_i8_u16_cfg0.json")))
    for k in ("kernel", "workload", "measured_at_commit", "commands", "fetch_size_kib_per_dispatch", "write_size_kib_per_dispatch",
              "copy_kernel", "scale", "traffic_bytes_per_launch", "algorithmic_bytes_per_launch"):
        assert k in side, k
    cp = side["copy_kernel"]
    assert abs(cp["bytes_read"] / 1024 / cp["fetch_size_kib_per_dispatch"] - side["scale"]["fetch_size"]) < 0.01
    assert abs(cp["bytes_written"] / 1024 / cp["write_size_kib_per_dispatch"] - side["scale"]["write_size"]) < 0.01
    want = (side["fetch_size_kib_per_dispatch"] * side["scale"]["fetch_size"] + side["write_size_kib_per_dispatch"] * side["scale"]["write_size"]) * 1024
    assert abs(side["traffic_bytes_per_launch"] - want) <= 1024
    assert side["algorithmic_bytes_per_launch"] == 32 * (2 * 4096 * 2560 + 6912 + 4 * 2560)
    assert 0.98 < side["traffic_bytes_per_launch"] / side["algorithmic_bytes_per_launch"] < 1.05
    assert all("bench.py" in c and c.startswith("rocprofv3 --pmc") for c in side["commands"])
