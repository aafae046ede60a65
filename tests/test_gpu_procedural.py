"""PROCEDURAL connectivity: rows (and weights) are regenerated for every spike instead of being stored.

The reference's own procedural strategies re-run the connectivity snippet with hiprand streams
(presynapticUpdateStrategySIMT.cc:391-560), so their synapses differ from every other backend's; what the feature
promises is that the network behaves like the one the same snippets would have *stored*.  That is testable exactly here:
a PROCEDURAL projection must deliver, synapse for synapse, what a SPARSE projection initialised on the device from the
same seed delivers — and that stored matrix is itself held to the snippets' distributions by tests/test_gpu_init.py.
"""
import numpy as np
import pytest

from genn_amd.genn_model import (GeNNModel, init_postsynaptic, init_sparse_connectivity, init_var, init_weight_update)

pytestmark = pytest.mark.gpu

LIF_SILENT = {"C": 1.0, "TauM": 20.0, "Vrest": -60.0, "Vreset": -60.0, "Vthresh": 1e9, "Ioffset": 0.0, "TauRefrac": 5.0}
LIF = {"C": 1.0, "TauM": 20.0, "Vrest": -60.0, "Vreset": -60.0, "Vthresh": -50.0, "Ioffset": 0.0, "TauRefrac": 2.0}


def _source(model, n, batch_size, fire_steps):
    """SpikeSourceArray in which neuron i of batch b fires once, at step fire_steps[b][i] (or never, if negative)."""
    fire = np.asarray(fire_steps)
    start = np.zeros((batch_size, n), np.uint32)
    end = np.zeros((batch_size, n), np.uint32)
    times = []
    for b in range(batch_size):
        for i in range(n):
            start[b, i] = len(times)
            if fire[b, i] >= 0:
                times.append(float(fire[b, i]))
            end[b, i] = len(times)
    src = model.add_neuron_population("S", n, "SpikeSourceArray", {}, {"startSpike": start, "endSpike": end})
    src.set_extra_global_param("spikeTimes", np.asarray(times + [0.0], np.float32))
    return src


def _pair(matrix_type, connect, weights, n_src, n_trg, fire, batch_size=1, seed=11):
    model = GeNNModel("float", "proc", batch_size=batch_size, dt=1.0)
    model.seed = seed
    src = _source(model, n_src, batch_size, fire)
    trg = model.add_neuron_population("T", n_trg, "LIF", LIF_SILENT, {"V": -60.0, "RefracTime": 0.0})
    if weights == "constant":
        wu = init_weight_update("StaticPulseConstantWeight", {"g": 0.375})
    else:
        wu = init_weight_update("StaticPulse", {}, {"g": weights})
    s = model.add_synapse_population("ST", matrix_type, src, trg, wu, init_postsynaptic("DeltaCurr"), init_sparse_connectivity(*connect))
    model.build()
    model.load()
    return model, s


@pytest.mark.parametrize("connect", [("FixedProbability", {"prob": 0.07}), ("FixedProbabilityNoAutapse", {"prob": 0.2}),
                                     ("FixedNumberPostWithReplacement", {"num": 37}), ("FixedNumberPostWithReplacement", {"num": 700})])
@pytest.mark.parametrize("weights", ["constant", "uniform", "normal", "number"])
def test_procedural_delivers_what_the_stored_matrix_delivers(connect, weights):
    n_src, n_trg, steps, B = 900, 900, 6, 2
    rng = np.random.default_rng(4)
    fire = rng.integers(-3, steps - 1, (B, n_src))            # about half the sources fire once, at a random step
    w = {"constant": "constant", "uniform": init_var("Uniform", {"min": -0.5, "max": 1.0}),
         "normal": init_var("Normal", {"mean": 0.1, "sd": 0.3}), "number": 0.625}[weights]
    stored, s_stored = _pair("SPARSE", connect, w, n_src, n_trg, fire, B)
    procedural, s_proc = _pair("PROCEDURAL", connect, w, n_src, n_trg, fire, B)
    assert "ind" not in s_proc.vars and "g" not in s_proc.vars          # nothing stored
    s_stored.pull_connectivity_from_device()
    ind, row_length = s_stored.ind_host, s_stored.row_length_host
    g = s_stored.vars["g"].pull_from_device().reshape(n_src, -1).astype(np.float64)
    events = 0
    for step in range(steps):
        stored.update_synapses()
        procedural.update_synapses()
        got = s_proc.vars["outPost"].pull_from_device().reshape(B, n_trg)
        want = s_stored.vars["outPost"].pull_from_device().reshape(B, n_trg)
        brute = np.zeros((B, n_trg))
        for b in range(B):
            for i in np.flatnonzero((fire[b] >= 0) & (fire[b] == step - 1)):
                np.add.at(brute[b], ind[i, :row_length[i]], g[i, :row_length[i]])
                events += int(row_length[i])
        peak = max(1.0, float(np.abs(brute).max()))
        assert np.abs(want - brute).max() <= 1e-5 * peak, f"step {step}: stored matrix against brute force"
        assert np.abs(got - brute).max() <= 1e-5 * peak, f"step {step}: procedural against brute force"
        if weights in ("constant", "number"):
            assert np.array_equal(got, want)           # sums of one value: exact in any order
        stored.update_neurons()
        procedural.update_neurons()
    assert events > 1000
    assert procedural.synaptic_event_count == stored.synaptic_event_count == events
    stored.unload()
    procedural.unload()


def test_procedural_recurrent_network_matches_stored_twin():
    """A recurrent LIF network (excitatory and inhibitory constant-weight projections, one postsynaptic model each)
    stepped 300 times: the procedural model and its stored twin must stay identical in every spike and every state value,
    through single steps and through run()."""
    def build(matrix_type):
        model = GeNNModel("float", "proc_net", dt=1.0)
        model.seed = 5
        e = model.add_neuron_population("E", 1600, "LIF", dict(LIF, Ioffset=0.56), {"V": init_var("Uniform", {"min": -60.0, "max": -50.0}), "RefracTime": 0.0})
        i = model.add_neuron_population("I", 400, "LIF", dict(LIF, Ioffset=0.56), {"V": init_var("Uniform", {"min": -60.0, "max": -50.0}), "RefracTime": 0.0})
        e.spike_recording_enabled = i.spike_recording_enabled = True
        for name, src, trg, w, tau, conn in (("EE", e, e, 0.05, 5.0, ("FixedProbabilityNoAutapse", {"prob": 0.05})),
                                            ("EI", e, i, 0.05, 5.0, ("FixedNumberPostWithReplacement", {"num": 20})),
                                            ("IE", i, e, -0.3, 10.0, ("FixedProbability", {"prob": 0.05})),
                                            ("II", i, i, -0.3, 10.0, ("FixedProbabilityNoAutapse", {"prob": 0.05}))):
            model.add_synapse_population(name, matrix_type, src, trg, init_weight_update("StaticPulseConstantWeight", {"g": w}),
                                         init_postsynaptic("ExpCurr", {"tau": tau}), init_sparse_connectivity(*conn))
        model.build()
        model.load(num_recording_timesteps=300)
        return model
    stored, procedural = build("SPARSE"), build("PROCEDURAL")
    for _ in range(100):
        stored.step_time()
        procedural.step_time()
    stored.run(200)
    procedural.run(200)
    stored.pull_recording_buffers_from_device()
    procedural.pull_recording_buffers_from_device()
    spikes = 0
    for name in ("E", "I"):
        a, b = stored.neuron_populations[name], procedural.neuron_populations[name]
        assert np.array_equal(a.vars["recordSpk"].view, b.vars["recordSpk"].view), f"rasters of {name} differ"
        for var in ("V", "RefracTime"):
            assert np.array_equal(a.vars[var].pull_from_device(), b.vars[var].pull_from_device()), f"{var} of {name} differs"
        spikes += len(a.spike_recording_data[0][1])
    assert spikes > 2000
    assert stored.synaptic_event_count == procedural.synaptic_event_count
    stored.unload()
    procedural.unload()
