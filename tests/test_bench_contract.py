"""bench.py's contract: one JSON line with the agreed fields; one GPU only."""
import json
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BENCH = os.path.join(ROOT, "bench.py")


def test_more_than_one_gpu_is_refused_with_a_message():
    done = subprocess.run([sys.executable, BENCH, "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert done.returncode == 2
    assert "one GPU only" in done.stderr and done.stdout.strip() == ""


@pytest.mark.gpu
def test_the_line_of_a_small_workload_has_every_field():
    """The 720p workload with three timed frames: the fields the contract names, the roofline and
    CPU-baseline objects, the figures this build adds beside them, and values that hang together."""
    done = subprocess.run([sys.executable, BENCH, "--config", "0", "--steps", "3", "--warmup", "2", "--headline-only", "--cpu-reps", "1"],
                          capture_output=True, text=True, timeout=600, cwd=ROOT)
    assert done.returncode == 0, done.stderr[-2000:]
    lines = [l for l in done.stdout.splitlines() if l.startswith("{")]
    assert len(lines) == 1
    d = json.loads(lines[0])
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                "vs_baseline", "dtype", "data", "config", "roofline", "cpu_baseline"):
        assert key in d, key
    assert d["n_gpus"] == 1 and d["steps"] == 3 and d["warmup"] == 2 and d["higher_is_better"] is True
    assert d["unit"] == "frames/s" and d["dtype"] == "f32" and d["data"] == "synthetic" and d["vs_baseline"] is None
    assert d["config"]["workload"] == "cfg0_100k_720p" and "model" not in d["config"]
    assert abs(d["value"] * d["ms_per_step"] / 1000.0 - 1.0) < 0.01            # frames/s and ms per frame of one measurement
    roof = d["roofline"]
    for key in ("kernel", "bound", "achieved", "peak", "unit", "frac", "traffic"):
        assert key in roof, key
    assert roof["bound"] in ("hbm", "mfma", "valu") and roof["kernel"].endswith("true>")      # the fp32 kernel was timed
    assert abs(roof["frac"] - roof["achieved"] / roof["peak"]) < 1e-3
    cpu = d["cpu_baseline"]
    for key in ("value", "unit", "cores", "kind", "sample"):
        assert key in cpu, key
    assert cpu["kind"] == "port" and cpu["cores"] >= 1 and cpu["value"] > 0
    assert d["ops_surface_image_identical"] is True
    assert d["config"]["two_frames_in_flight"]["images_identical"] is True
    assert d["two_frames_in_flight_fps"] > 0 and d["fast_mode_fps"] > 0 and d["blocking_readback_ms_per_frame"] > 0
    assert set(d["stages"]) == {"preprocess", "sort", "ranges", "readback", "blend"}
