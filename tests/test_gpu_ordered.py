"""Ordered accumulation (validation mode): every postsynaptic element is summed in the order of the reference's
SingleThreadedCPU backend — projections one after another, spikes in queue order, synapses in ascending position
(src/genn/backends/single_threaded_cpu/backend.cc:1884-1929) — without atomics.  In this mode a FREE-RUNNING network must
stay bit-identical to the oracle in everything: rasters, neuron state, outPost, every slot of the dendritic-delay rings,
plastic weights and traces.  That is the evidence that the default mode's differences (within 1e-5, rasters that part
once a threshold crossing flips) come from the order of its fp32 atomic adds and from nothing else."""
import numpy as np
import pytest

from genn_amd import configs
from genn_amd.genn_model import model_from_net
from oracle.genn_cpu import OracleNet
from parity import compare_state

pytestmark = pytest.mark.gpu


def free_run_identical(net, steps, plastic=(), use_graph=True):
    model = model_from_net(net, ordered=True)
    model.load(num_recording_timesteps=steps)
    info = model.runner_info()
    assert info["ordered_accumulation"] and not info["single_launch_step"] and not info["resident_plan"]
    oracle = OracleNet(net, num_recording_timesteps=steps,
                       col_stride={name: model.synapse_populations[name].col_stride for name in plastic} or None)
    if use_graph:
        model.run(steps)
    else:
        for _ in range(steps):
            model.step_time()
    oracle.run(steps)
    model.pull_recording_buffers_from_device()
    spikes = 0
    for p in net.pops:
        got = model.neuron_populations[p.name].vars["recordSpk"].view
        want = oracle.record(p.name, steps)
        words = (p.n + 31) // 32
        if not np.array_equal(got, want):
            first = int(np.nonzero((got.reshape(steps, words) != want.reshape(steps, words)).any(axis=1))[0][0])
            raise AssertionError(f"raster of {p.name} differs first at step {first}")
        spikes += int(np.unpackbits(np.ascontiguousarray(want).view(np.uint8)).sum())
    compare_state(net, model, oracle, f"after {steps} free-running steps", exact=True)
    assert model.synaptic_event_count == oracle.events()
    return model, oracle, spikes


def test_ordered_izhikevich_free_run():
    """Configuration-3 shape (multapses, mixed-sign weights of many values, DeltaCurr): 300 free-running steps, through the
    population bursts in which the default mode's rasters part from the oracle's."""
    net = configs.izhikevich_fanout(n=20000, fanout=100, steps=300)
    model, oracle, spikes = free_run_identical(net, 300)
    assert spikes > 3000
    model.unload()


def test_ordered_microcircuit_free_run():
    """Configuration-2 shape at 5 % of the neurons with full in-degree: 54 projections fused into 8 rings of 43 slots; every
    slot of every ring bit-identical after 1500 free-running steps (150 ms)."""
    net = configs.potjans(neuron_scale=0.05, connectivity_scale=1.0, steps=1500)
    model, oracle, spikes = free_run_identical(net, 1500)
    assert spikes > 1000
    model.unload()


@pytest.mark.parametrize("rule", ["stdp_trace", "stdp_additive"])
def test_ordered_plastic_free_run(rule):
    """Configuration-4 shape: plastic E->E next to static projections into shared postsynaptic models; weights, traces and
    both column views bit-identical after 300 free-running steps."""
    net = configs.plastic_stdp(n=5000, n_src=100, steps=300, fan=250, src_fan=50, rule=rule)
    model, oracle, spikes = free_run_identical(net, 300, plastic=("EE",))
    assert spikes > 3000
    model.unload()


def test_ordered_balanced_network_stepwise_and_axonal_delay():
    """Configuration-1 shape with axonal delay slots on two projections, stepped one launch sequence at a time."""
    net = configs.vogels_abbott(n=2000, steps=400, p=0.05, axonal_delays={"EI": 3, "IE": 1})
    model, oracle, spikes = free_run_identical(net, 400, use_graph=False)
    assert spikes > 500
    model.unload()


def test_default_mode_is_not_bit_identical_where_ordered_mode_is():
    """The same configuration-3-shaped network in the default mode: input sums agree with the oracle's only to rounding
    (some element differs in its last bits once thousands of differently-valued weights have been added by atomics),
    which is exactly the difference ordered accumulation removes."""
    net = configs.izhikevich_fanout(n=20000, fanout=100, steps=60)
    model = model_from_net(net)
    model.load(num_recording_timesteps=60)
    oracle = OracleNet(net, num_recording_timesteps=60)
    differing = 0
    for step in range(60):
        model.update_synapses()
        oracle.update_synapses()
        got, want = model.synapse_populations["NN"].vars["outPost"].pull_from_device(), oracle.out_post("NN")
        differing += int(np.count_nonzero(got != want))
        peak = max(1e-3, float(np.abs(want).max()))
        assert float(np.abs(got.astype(np.float64) - want).max()) <= 1e-5 * peak
        want[:] = got
        model.update_neurons()
        oracle.update_neurons()
        assert np.array_equal(model.neuron_populations["N"].current_spikes[0], oracle.spikes("N"))
        for k, name in enumerate(("V", "U")):
            oracle.var("N", k)[:] = model.neuron_populations["N"].vars[name].pull_from_device()
    assert differing > 0, "atomic order happened to reproduce every sum: pick a busier network"
    model.unload()
