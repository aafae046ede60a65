"""Timing counters as the user sees them (generateRunner.cc:159-174, runtime.h:324-333, pygenn/genn_model.py:292-326),
modelled on the reference's tests/features/test_model_timing.py: with timing enabled every documented counter is
accessible, non-negative and accumulates over a simulation — under every launch plan, through the Python host layer and
through the reference's own Runtime on the backend adapter."""
import os
import re
import shutil
import subprocess
import sys
import tempfile

import numpy as np
import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
sys.path.insert(0, os.path.join(HERE, "golden"))

from genn_amd import configs  # noqa: E402
from genn_amd.genn_model import model_from_net  # noqa: E402
from genn_amd.netspec import write_netspec  # noqa: E402

pytestmark = pytest.mark.gpu

COUNTERS = ("neuron_update_time", "init_time", "init_sparse_time", "presynaptic_update_time", "postsynaptic_update_time", "synapse_dynamics_time")


def _check_accumulation(model, advance):
    initial = [getattr(model, c) for c in COUNTERS]
    advance()
    final = [getattr(model, c) for c in COUNTERS]
    for name, a, b in zip(COUNTERS, initial, final):
        assert np.isfinite(b) and b >= 0.0, name
        assert b >= a, f"{name} must accumulate"
    return dict(zip(COUNTERS, final))


def test_counters_of_a_plastic_network():
    """Two LIF populations, built-in STDP on a SPARSE projection (the reference test's model): three kernels per step, one
    counter each; learnPost runs every step, so postsynaptic_update_time grows too."""
    net = configs.plastic_stdp(n=2000, n_src=100, steps=200, fan=100, src_fan=50, rule="stdp_additive")
    model = model_from_net(net)
    model.timing_enabled = True
    model.load(num_recording_timesteps=200)
    first = _check_accumulation(model, lambda: [model.step_time() for _ in range(100)])
    assert first["neuron_update_time"] > 0 and first["presynaptic_update_time"] > 0 and first["postsynaptic_update_time"] > 0
    assert first["init_time"] > 0
    second = _check_accumulation(model, lambda: model.run(100))          # run() steps kernel by kernel while timing is enabled
    for c in ("neuron_update_time", "presynaptic_update_time", "postsynaptic_update_time"):
        assert second[c] > first[c], c
    # the counters are device time of the kernels: a hundred steps of three short kernels cannot add up to a second
    assert second["neuron_update_time"] + second["presynaptic_update_time"] + second["postsynaptic_update_time"] < 1.0
    model.unload()


def test_counters_under_the_single_launch_and_resident_plans():
    """The microcircuit shape takes the single-launch step (and the resident plan for run()): with timing enabled run() steps
    launch by launch, and the one kernel of a step is reported as neuron update time."""
    net = configs.potjans(neuron_scale=0.05, connectivity_scale=1.0, steps=300)
    model = model_from_net(net)
    model.timing_enabled = True
    model.load(num_recording_timesteps=300)
    info = model.runner_info()
    assert info["single_launch_step"] and info["resident_plan"]
    first = _check_accumulation(model, lambda: [model.step_time() for _ in range(100)])
    assert first["neuron_update_time"] > 0 and first["presynaptic_update_time"] == 0.0 and first["postsynaptic_update_time"] == 0.0
    second = _check_accumulation(model, lambda: model.run(200))
    assert second["neuron_update_time"] > first["neuron_update_time"]
    model.set_timing(False)
    frozen = model.neuron_update_time
    model.run(50)
    model.synchronize()
    assert model.neuron_update_time == frozen, "counters only run while timing is enabled"
    model.unload()


def test_counters_through_the_reference_runtime():
    """ModelSpec::setTimingEnabled through the adapter: the generated runner's exported doubles, read by
    Runtime::get*Time (runtime.h:324-333)."""
    driver = os.path.join(ROOT, "oracle", "_ref", "mi355x_driver")
    if not os.path.exists(driver):
        pytest.skip("oracle/_ref/mi355x_driver is not built")
    from cases import CASES
    net, snap = CASES["stdp_additive_small"]()
    net.snap = snap
    tmp = tempfile.mkdtemp(prefix="adapter_timing_")
    try:
        spec, work, out = (os.path.join(tmp, d) for d in ("spec", "work", "out"))
        for d in (work, out):
            os.makedirs(d)
        write_netspec(net, spec)
        res = subprocess.run([driver, spec, work, out, "--timing"], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=300)
        assert res.returncode == 0, res.stdout[-3000:]
        m = re.search(r"timers init (\S+) initSparse (\S+) neuronUpdate (\S+) presynapticUpdate (\S+) postsynapticUpdate (\S+)", res.stdout)
        assert m, res.stdout[-2000:]
        init, sparse, neuron, pre, post = (float(x) for x in m.groups())
        assert init > 0 and sparse > 0 and neuron > 0 and pre > 0 and post > 0
        assert neuron + pre + post < 1.0
    finally:
        shutil.rmtree(tmp, ignore_errors=True)


def test_counters_of_generated_kernels_through_the_reference_runtime():
    """The same counters when the step's kernels are generated from model code: events around each update's launches, read
    in stepTime after the step has been synchronised (as the reference's device backends do), and per custom update group
    inside its update function."""
    driver = os.path.join(ROOT, "oracle", "_ref", "mi355x_driver")
    if not os.path.exists(driver):
        pytest.skip("oracle/_ref/mi355x_driver is not built")
    from cases import CASES
    net, snap = CASES["custom_update_small"]()
    net.snap = snap
    tmp = tempfile.mkdtemp(prefix="adapter_timing_generated_")
    try:
        spec, work, out = (os.path.join(tmp, d) for d in ("spec", "work", "out"))
        for d in (work, out):
            os.makedirs(d)
        write_netspec(net, spec)
        res = subprocess.run([driver, spec, work, out, "--timing"], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=300)
        assert res.returncode == 0, res.stdout[-3000:]
        m = re.search(r"timers init (\S+) initSparse (\S+) neuronUpdate (\S+) presynapticUpdate (\S+) postsynapticUpdate (\S+)", res.stdout)
        assert m, res.stdout[-2000:]
        init, sparse, neuron, pre, post = (float(x) for x in m.groups())
        assert init > 0 and sparse > 0 and neuron > 0 and pre > 0 and post > 0
        # 200 steps of three kernels of a few microseconds each
        assert 200 * 1e-6 < neuron < 0.5 and 200 * 1e-6 < pre < 0.5 and 200 * 1e-6 < post < 0.5
        custom = {g: (float(a), float(b)) for g, a, b in re.findall(r"timers customUpdate (\S+) (\S+) transpose (\S+)", res.stdout)}
        assert set(custom) == {"Homeostasis", "Decay", "Reduce"}
        assert all(1e-6 < t < 0.5 for t, _ in custom.values())
        assert custom["Decay"][1] > 1e-6 and custom["Reduce"][1] < 1e-4        # only Decay transposes
        # the rasters are those of the untimed run
        golden = np.load(os.path.join(HERE, "golden", "custom_update_small.npz"))
        for p in net.pops:
            got = np.fromfile(os.path.join(out, f"{p.name}.spikes.u32"), np.uint32).reshape(-1, 2)
            assert np.array_equal(got, golden[f"spikes.{p.name}"])
    finally:
        shutil.rmtree(tmp, ignore_errors=True)


def test_profiler_ranges_nest_and_cost_nothing_without_a_profiler():
    """gennmi_profiler_range_push / _pop (roctx ranges when libroctx64 can be loaded, nothing otherwise): always GENNMI_OK,
    nesting as generateRunner.cc:275-297 nests them."""
    from genn_amd import _abi
    lib = _abi.load()
    for name in (b"stepTime", b"updateSynapses"):
        assert lib.gennmi_profiler_range_push(name) == 0
    assert lib.gennmi_profiler_range_pop() == 0 and lib.gennmi_profiler_range_pop() == 0
    assert lib.gennmi_profiler_range_push(None) == 0
