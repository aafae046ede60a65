"""The benchmark's output contract, on the default workload: one JSON line with the headline metric, the roofline of the
dominant kernel measured inside the run, and a CPU baseline timed beside it."""
import json
import os
import subprocess
import sys

import pytest

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_default_bench_line():
    res = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--steps", "2000", "--warmup", "500", "--cpu-steps", "300",
                          "--reference-steps", "0", "--secondary-steps", "300"], stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, timeout=280, cwd=ROOT)
    assert res.returncode == 0, res.stderr[-2000:]
    lines = [line for line in res.stdout.splitlines() if line.strip()]
    assert len(lines) == 1, "exactly one line on stdout"
    out = json.loads(lines[0])
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling", "vs_baseline",
                "dtype", "data", "config", "roofline", "cpu_baseline"):
        assert key in out, key
    assert out["metric"] == "synaptic_events_per_s" and out["n_gpus"] == 1 and out["steps"] == 2000 and out["warmup"] == 500
    assert out["higher_is_better"] is True and out["vs_baseline"] is None and out["data"] == "synthetic" and out["dtype"] == "f32"
    assert "workload" in out["config"] and "model" not in out["config"]
    assert out["config"]["neurons"] == 77169 and out["config"]["synapses"] == 298624465
    roof = out["roofline"]
    assert roof["bound"] == "hbm" and roof["unit"] == "GB/s" and roof["peak"] == 8000.0
    assert abs(roof["frac"] - roof["achieved"] / roof["peak"]) < 1e-4 and 0.0 < roof["frac"] < 1.0
    assert roof["traffic"] is None or roof["traffic"] > 0
    cpu = out["cpu_baseline"]
    assert cpu["kind"] in ("port", "reference") and cpu["cores"] == 1 and cpu["value"] > 0 and cpu["unit"] == "events/s" and cpu["sample"]
    # whole-job throughput and step time are two views of the same clock
    assert abs(out["value"] - out["events_per_step"] / (out["ms_per_step"] * 1e-3)) <= 0.02 * out["value"]
    assert out["value"] > 10 * cpu["value"]
    # the bandwidth-bound configuration beside the headline one, with a roofline of its own
    sec = out["secondary"]
    assert "error" not in sec, sec
    assert sec["config"]["neurons"] == 1_000_000 and sec["config"]["synapses"] == 1_000_000_000 and sec["steps"] == 300
    assert sec["roofline"]["bound"] == "hbm" and 0.0 < sec["roofline"]["frac"] < 1.0
    assert "steady_state" not in out        # (a run of 2000 steps is the running network already)


def test_short_bench_line_carries_the_running_network():
    """The command the round's driver runs times 20 steps from t = 0; the line then also holds a `steady_state` block
    measured in the same process (here shortened), whose step time is the running network's."""
    res = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "1", "--steps", "20", "--warmup", "5", "--cpu-steps", "100",
                          "--reference-steps", "0", "--secondary-steps", "0", "--steady-steps", "3000", "--steady-warmup", "1000"],
                         stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, timeout=280, cwd=ROOT)
    assert res.returncode == 0, res.stderr[-2000:]
    out = json.loads([line for line in res.stdout.splitlines() if line.strip()][-1])
    assert out["steps"] == 20 and out["warmup"] == 5 and "secondary" not in out
    steady = out["steady_state"]
    assert steady["steps"] == 3000 and steady["warmup"] == 1000
    roof = steady["roofline"]
    assert roof["bound"] == "hbm" and abs(roof["frac"] - roof["achieved"] / roof["peak"]) < 1e-4 and 0.0 < roof["frac"] < 1.0
    # a step of the running network is shorter than one of the first 25 steps, which include the launch's start-up
    assert steady["us_per_step"] < out["ms_per_step"] * 1e3
    assert abs(steady["events_per_s"] - steady["events_per_step"] / (steady["us_per_step"] * 1e-6)) <= 0.02 * steady["events_per_s"]
