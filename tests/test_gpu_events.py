"""Spike-like events and graded synapses (StaticGraded, weightUpdateModels.h:308-319) on the GPU against the CPU oracle,
whose restatement of this path is pinned bit for bit by the fixture the reference's own CPU backend wrote
(tests/golden/graded_small.npz, tests/test_oracle_golden.py).

Held to: event queues and spike queues identical, in ascending neuron order, at every step; state and accumulators within
1e-5 (the GPU adds the releases with fp32 atomics in arbitrary order, the reference adds them in double, in row order);
event counts equal.
"""
import numpy as np
import pytest

from genn_amd import configs
from genn_amd.genn_model import model_from_net
from oracle.genn_cpu import OracleNet
from parity import compare_state

pytestmark = pytest.mark.gpu

GRADED = ("AB_graded", "AA_graded", "CB_graded")


def _event_queue(model, name):
    s = model.synapse_populations[name]
    e = s.src.event_thresholds.index(float(s.wu.params["Epre"]))
    B, n = model.batch_size, s.src.num_neurons
    cnt = s.src.vars[f"spkCntEvent{e}"].pull_from_device()
    queue = s.src.vars[f"spkEvent{e}"].pull_from_device().reshape(B, n)
    return [queue[b, :cnt[b]].copy() for b in range(B)]


def _lock_step(net, steps, batch_size=1, check_every=10):
    model = model_from_net(net, batch_size=batch_size)
    model.load(num_recording_timesteps=steps)
    info = model.runner_info()
    assert not info["single_launch_step"] and not info["resident_plan"]
    oracle = OracleNet(net, num_recording_timesteps=steps)
    events = spikes = 0
    for step in range(steps):
        model.step_time()
        oracle.step()
        for name in GRADED:
            want = oracle.spike_events(name)
            assert np.all(np.diff(want.astype(np.int64)) > 0)
            for b, got in enumerate(_event_queue(model, name)):
                assert np.array_equal(got, want), f"step {step}: event queue of {name}, batch {b} ({len(got)} vs {len(want)})"
            events += len(want)
        for p in net.pops:
            want = oracle.spikes(p.name)
            for b, got in enumerate(model.neuron_populations[p.name].current_spikes):
                assert np.array_equal(got, want), f"step {step}: spike queue of {p.name}, batch {b}"
            spikes += len(want)
        if (step + 1) % check_every == 0 and batch_size == 1:
            compare_state(net, model, oracle, f"step {step}", exact=False)
    assert model.synaptic_event_count == batch_size * oracle.events()
    return model, oracle, events, spikes


def test_graded_synapses_match_the_oracle():
    net = configs.graded()
    model, oracle, events, spikes = _lock_step(net, net.steps)
    assert events > 10000 and spikes > 300
    model.unload()


def test_graded_synapses_batched():
    """Every batch starts from the same state and has its own event queues, V and accumulators."""
    net = configs.graded(steps=60)
    model, oracle, events, spikes = _lock_step(net, 60, batch_size=3)
    for p in net.pops:
        got = model.neuron_populations[p.name].vars["V"].pull_from_device().reshape(3, p.n)
        for b in range(3):
            assert np.abs(got[b] - oracle.var(p.name, 0)).max() <= 1e-5 * 70.0
    model.unload()


def test_event_queues_across_many_blocks():
    """20,000 and 40,000 neurons: 79 and 157 blocks per population, so the queue offsets cross the boundary between the
    groups of 64 blocks whose totals are published separately; most of population A is above the threshold of one of its
    two event conditions at any time."""
    net = configs.graded(n_a=20000, n_b=40000, n_c=700, steps=40)
    model, oracle, events, spikes = _lock_step(net, 40, check_every=20)
    assert events > 500000
    model.unload()


def test_graded_synapses_through_run():
    """The same network stepped by run() (replayed graphs of the separate launches) ends in the same state."""
    net = configs.graded(steps=230)
    model = model_from_net(net)
    model.load(num_recording_timesteps=230)
    oracle = OracleNet(net, num_recording_timesteps=230)
    model.run(230)
    oracle.run(230)
    model.pull_recording_buffers_from_device()
    for p in net.pops:
        assert np.array_equal(model.neuron_populations[p.name].vars["recordSpk"].view, oracle.record(p.name, 230)), f"raster of {p.name}"
    for name in GRADED:
        assert np.array_equal(_event_queue(model, name)[0], oracle.spike_events(name))
    compare_state(net, model, oracle, "after run(230)", exact=False)
    assert model.synaptic_event_count == oracle.events()
    model.unload()


# ---- presynaptic ("reverse") output: addToPre --------------------------------------------------------------------------
def _reverse_lock_step(net, steps, exact):
    from parity import assert_close
    model = model_from_net(net)
    model.load(num_recording_timesteps=steps)
    info = model.runner_info()
    assert not info["single_launch_step"] and not info["resident_plan"]
    oracle = OracleNet(net, num_recording_timesteps=steps)
    spikes, fed_back = 0, 0.0
    for step in range(steps):
        model.update_synapses()
        oracle.update_synapses()
        for name in ("AB_reverse", "BA_reverse"):
            got = model.synapse_populations[name].vars["outPre"].pull_from_device()
            want = oracle.out_pre(name)
            assert_close(got, want, f"step {step}: outPre of {name}", exact, accumulator=True)
            fed_back += float(np.abs(want).sum())
        model.update_neurons()
        oracle.update_neurons()
        for name in ("AB_reverse", "BA_reverse"):
            assert not model.synapse_populations[name].vars["outPre"].pull_from_device().any(), "outPre is consumed by the neuron update"
        for p in net.pops:
            want = oracle.spikes(p.name)
            assert np.array_equal(model.neuron_populations[p.name].current_spikes[0], want), f"step {step}: spike queue of {p.name}"
            spikes += len(want)
        if (step + 1) % 10 == 0:
            compare_state(net, model, oracle, f"step {step}", exact=False)
    assert model.synaptic_event_count == oracle.events()
    assert spikes > 500 and fed_back > 100.0
    model.unload()


def test_reverse_output_exact_with_dyadic_weights():
    """Weights that are multiples of 1/8: the sum of a row is exact in any order and outPre starts every step at zero, so
    outPre must equal the oracle's bit for bit although the GPU adds a row's weights by wavefront reduction.  (The
    forward projections' ExpCurr accumulators carry a decayed remainder, so they stay within tolerance only.)"""
    net = configs.reverse()
    for s in net.syns:
        s.g = (np.round(s.g * 8.0) / 8.0).astype(np.float32)
    _reverse_lock_step(net, 100, exact=True)


def test_reverse_output_matches_the_oracle():
    """The fixture's network (arbitrary weights): identical spike queues over the first 100 steps, outPre and state within
    1e-5 (a row's weights are summed in a different order)."""
    net = configs.reverse()
    _reverse_lock_step(net, 100, exact=False)


def test_spike_event_recording():
    """Recorded spike-like events (one bitfield per event queue, laid out like the spike recording) against the oracle,
    through single steps and a replayed run, for every batch."""
    net = configs.graded(steps=120)
    B = 2
    model = model_from_net(net, batch_size=B)
    for p in model.neuron_populations.values():
        p.spike_event_recording_enabled = True
    model.load(num_recording_timesteps=120)
    oracle = OracleNet(net, num_recording_timesteps=120)
    for _ in range(20):
        model.step_time()
    model.run(100)
    oracle.run(120)
    model.pull_recording_buffers_from_device()
    total = 0
    for name in GRADED:
        src = model.synapse_populations[name].src
        words = (src.num_neurons + 31) // 32
        e = src.event_thresholds.index(float(model.synapse_populations[name].wu.params["Epre"]))
        got = src.vars[f"recordSpkEvent{e}"].view.reshape(120, B, words)
        want = oracle.event_record(name, 120).reshape(120, words)
        for b in range(B):
            assert np.array_equal(got[:, b], want), f"recorded events of {name}, batch {b}"
        times, ids = model.synapse_populations[name].pre_spike_event_recording_data[0]
        assert len(ids) == int(np.unpackbits(want.view(np.uint8)).sum())
        total += len(ids)
    assert total > 5000
    model.unload()
