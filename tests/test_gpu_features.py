"""The reference's feature tests for the hot path (tests/features/test_event_propagation.py,
test_recording.py), restated against the MI355X engine.  They pin the path with closed-form
answers: binary decode of one-hot spike sources, a dendritic-delay ramp that must sum to
exactly 10.0 at step 11, the Sobel fixtures of the Toeplitz test, and a decode through the
column remap.  The reference reads a custom "x = Isyn" neuron; here the same quantity is read
as outPost between updateSynapses and updateNeurons (with DeltaCurr, Isyn IS outPost)."""
import os

import numpy as np
import pytest

from genn_amd.genn_model import GeNNModel, init_postsynaptic, init_toeplitz_connectivity, init_weight_update

pytestmark = pytest.mark.gpu

FIXTURES = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "reference_fixtures")
LIF = {"C": 1.0, "TauM": 20.0, "Vrest": -60.0, "Vreset": -60.0, "Vthresh": 1e9, "Ioffset": 0.0, "TauRefrac": 5.0}


def _silent_pop(model, name, n):
    return model.add_neuron_population(name, n, "LIF", LIF, {"V": np.full(n, -60.0, np.float32), "RefracTime": np.zeros(n, np.float32)})


def _decoder_lists(n_src=16, n_trg=4):
    pre, post = [], []
    for i in range(n_src):
        for j in range(n_trg):
            if ((i + 1) & (1 << j)) != 0:
                pre.append(i)
                post.append(j)
    return np.asarray(pre), np.asarray(post)


# tests/features/test_event_propagation.py:65-260
def test_forward(make_model):
    model = make_model("float", "test_forward", dt=1.0)
    ss = model.add_neuron_population("SpikeSource", 16, "SpikeSourceArray", {},
                                     {"startSpike": np.arange(16), "endSpike": np.arange(1, 17)})
    ss.set_extra_global_param("spikeTimes", np.arange(16.0))
    pre, post = _decoder_lists()
    outputs = []
    for name, hint, tps in (("Sparse", "POSTSYNAPTIC", 1), ("SparsePreSpan", "PRESYNAPTIC", 1),
                            ("SparseHybrid", "PRESYNAPTIC", 2), ("SparseWave", "WAVE", 1)):
        n = _silent_pop(model, "Post" + name, 4)
        s = model.add_synapse_population(name + "Synapse", "SPARSE", ss, n,
                                         init_weight_update("StaticPulse", {}, {"g": 1.0}), init_postsynaptic("DeltaCurr"))
        s.set_sparse_connections(pre, post)
        s.parallelism_hint = hint
        s.num_threads_per_spike = tps
        outputs.append(s)
    # the reference's other decoder projections: constant weight (SPARSE, BITMASK), DENSE with individual weights
    n = _silent_pop(model, "PostSparseConstantWeight", 4)
    s = model.add_synapse_population("SparseConstantWeightSynapse", "SPARSE", ss, n,
                                     init_weight_update("StaticPulseConstantWeight", {"g": 1.0}), init_postsynaptic("DeltaCurr"))
    s.set_sparse_connections(pre, post)
    outputs.append(s)
    n = _silent_pop(model, "PostBitmask", 4)
    s = model.add_synapse_population("BitmaskSynapse", "BITMASK", ss, n,
                                     init_weight_update("StaticPulseConstantWeight", {"g": 1.0}), init_postsynaptic("DeltaCurr"))
    s.set_sparse_connections(pre, post)
    outputs.append(s)
    dense = np.zeros((16, 4), np.float32)
    dense[pre, post] = 1.0
    n = _silent_pop(model, "PostDense", 4)
    s = model.add_synapse_population("DenseSynapse", "DENSE", ss, n,
                                     init_weight_update("StaticPulse", {}, {"g": dense.flatten()}), init_postsynaptic("DeltaCurr"))
    outputs.append(s)
    model.build()
    model.load()
    place = 2 ** np.arange(4)
    while model.timestep < 16:
        model.update_synapses()
        for s in outputs:
            x = s.vars["outPost"].pull_from_device()
            value = np.sum(place[np.isclose(np.ones(4), x)])
            # spikes emitted in timestep n arrive in timestep n+1
            expect = model.timestep if model.timestep > 0 else 0
            assert value == expect, f"{s.name} decoding incorrect ({value} rather than {expect})"
        model.update_neurons()


# tests/features/test_event_propagation.py:262-329 (batch sizes 1 and 5, conftest.py:38-64)
@pytest.mark.parametrize("batch_size", [1, 5])
def test_forward_den_delay(make_model, batch_size):
    model = make_model("float", "test_forward_den_delay", dt=1.0, batch_size=batch_size)
    ss = model.add_neuron_population("SpikeSource", 10, "SpikeSourceArray", {},
                                     {"startSpike": np.arange(10), "endSpike": np.arange(1, 11)})
    ss.set_extra_global_param("spikeTimes", np.arange(10.0))
    delay = np.arange(9, -1, -1)
    outputs = []
    for name, hint in (("Sparse", "POSTSYNAPTIC"), ("SparsePreSpan", "PRESYNAPTIC")):
        n = _silent_pop(model, "Post" + name, 1)
        s = model.add_synapse_population(name + "Synapse", "SPARSE", ss, n,
                                         init_weight_update("StaticPulseDendriticDelay", {}, {"g": 1.0, "d": 0}),
                                         init_postsynaptic("DeltaCurr"))
        s.max_dendritic_delay_timesteps = 10
        s.set_sparse_connections(np.arange(10), np.zeros(10, dtype=int))
        s.set_var_coo("d", delay)
        s.parallelism_hint = hint
        outputs.append(s)
    model.build()
    model.load()
    # Isyn of the neuron update in timestep n is outPost + the ring's front slot; the neuron kernel
    # folds the front slot in and DeltaCurr clears it, so observe the front slot before it runs
    while model.timestep < 11:
        model.update_synapses()
        ptr = (model.timestep + 1) % 10
        correct = 10.0 if model.timestep == 10 else 0.0
        for s in outputs:
            ring = s.vars["denDelay"].pull_from_device().reshape(batch_size, 10, 1)
            assert np.allclose(ring[:, ptr, 0], correct), f"{s.name} decoding incorrect ({ring[:, ptr, 0]} rather than {correct})"
        model.update_neurons()
        for s in outputs:
            assert s.vars["denDelayPtr"].pull_from_device()[0] == ptr


# tests/features/test_event_propagation.py:387-485 with the reference's own fixtures
def test_forward_kernel(make_model):
    vertical = np.asarray([[1.0, 0.0, -1.0], [2.0, 0.0, -2.0], [1.0, 0.0, -1.0]])
    horizontal = np.asarray([[1.0, 2.0, 1.0], [0.0, 0.0, 0.0], [-1.0, -2.0, -1.0]])
    model = make_model("float", "test_forward_kernel", dt=1.0)
    pattern = np.load(os.path.join(FIXTURES, "test_pattern.npy"))
    end = np.cumsum(np.bincount(pattern, minlength=64 * 64))
    start = np.concatenate(([0], end[:-1]))
    pre = model.add_neuron_population("SpikeSource", 64 * 64, "SpikeSourceArray", {}, {"startSpike": start, "endSpike": end})
    pre.set_extra_global_param("spikeTimes", np.zeros(len(pattern)))
    params = {"conv_kh": 3, "conv_kw": 3, "conv_ih": 64, "conv_iw": 64, "conv_ic": 1, "conv_oh": 62, "conv_ow": 62, "conv_oc": 1}
    syn = {}
    for name, kern in (("Horiz", horizontal), ("Vert", vertical)):
        post = _silent_pop(model, "Post" + name, 62 * 62)
        syn[name] = model.add_synapse_population("Toeplitz" + name, "TOEPLITZ", pre, post,
                                                 init_weight_update("StaticPulse", {}, {"g": kern.flatten()}),
                                                 init_postsynaptic("DeltaCurr"), init_toeplitz_connectivity("Conv2D", params))
    model.build()
    model.load()
    model.step_time()
    model.update_synapses()
    assert np.allclose(syn["Horiz"].vars["outPost"].pull_from_device(), np.load(os.path.join(FIXTURES, "horizontal_output.npy")))
    assert np.allclose(syn["Vert"].vars["outPost"].pull_from_device(), np.load(os.path.join(FIXTURES, "vertical_output.npy")))


# learnPost through the column remap, as a decode in the style of test_event_propagation.py:848-955:
# postsynaptic spike j must touch exactly the synapses {i -> j : bit i of j+1 set}
def test_learn_post_decode(make_model):
    model = make_model("float", "test_learn_post", dt=1.0)
    pre_pop = _silent_pop(model, "Pre", 4)
    post_pop = model.add_neuron_population("SpikeSource", 16, "SpikeSourceArray", {},
                                           {"startSpike": np.arange(16), "endSpike": np.arange(1, 17)})
    post_pop.set_extra_global_param("spikeTimes", np.arange(16.0))
    post_inds, pre_inds = _decoder_lists()        # (source index 0..15, bit 0..3) -> post j, pre i
    stdp = {"tauPlus": 1e30, "tauMinus": 1e30, "aPlus": 1.0, "aMinus": 0.0, "wMin": 0.0, "wMax": 100.0}
    s = model.add_synapse_population("Plastic", "SPARSE", pre_pop, post_pop,
                                     init_weight_update("STDPTrace", stdp, {"g": 0.0}, {"preTrace": 1.0}, {"postTrace": 0.0}),
                                     init_postsynaptic("DeltaCurr"))
    s.set_sparse_connections(pre_inds, post_inds)
    model.build()
    model.load()
    col_length = s.vars["colLength"].pull_from_device()
    assert np.array_equal(col_length, [bin((j + 1) & 15).count("1") for j in range(16)])
    place = 2 ** np.arange(4)
    seen = np.zeros((4, s.row_stride), np.float32)
    while model.timestep < 16:
        model.step_time()
        g = s.vars["g"].pull_from_device().reshape(4, s.row_stride)
        changed = (g != seen)
        seen = g.copy()
        rows, cols = np.nonzero(changed)
        value = int(np.sum(place[rows]))
        assert value == model.timestep - 1, f"learnPost decoding incorrect ({value} rather than {model.timestep - 1})"
        if len(rows):
            assert np.all(s.ind_host[rows, cols] == model.timestep - 2)
            assert np.allclose(g[rows, cols], 1.0)


# tests/features/test_recording.py:56-134 — bitfield round trip, batched, ragged population size
@pytest.mark.parametrize("batch_size", [1, 3])
def test_spike_recording(make_model, batch_size):
    n = 100
    rng = np.random.default_rng(7)
    model = make_model("float", "test_spike_recording", dt=1.0, batch_size=batch_size)
    spikes = [[np.sort(rng.choice(50, rng.integers(0, 6), replace=False)).astype(np.float32) for _ in range(n)] for _ in range(batch_size)]
    times = np.concatenate([np.concatenate(b) if any(len(x) for x in b) else np.zeros(0, np.float32) for b in spikes])
    counts = np.array([[len(x) for x in b] for b in spikes]).reshape(-1)
    end = np.cumsum(counts).astype(np.uint32).reshape(batch_size, n)
    start = (end.reshape(-1) - counts).astype(np.uint32).reshape(batch_size, n)
    pop = model.add_neuron_population("SpikeSource", n, "SpikeSourceArray", {}, {"startSpike": start, "endSpike": end})
    pop.set_extra_global_param("spikeTimes", times)
    pop.spike_recording_enabled = True
    model.build()
    model.load(num_recording_timesteps=50)
    for _ in range(50):
        model.step_time()
    model.pull_recording_buffers_from_device()
    data = pop.spike_recording_data
    for b in range(batch_size):
        rec_t, rec_id = data[b]
        want = sorted((float(t), i) for i in range(n) for t in spikes[b][i])
        got = sorted(zip(rec_t.tolist(), rec_id.tolist()))
        assert got == want


@pytest.mark.parametrize("count", [1, 3, 4, 1023, 1 << 20])
def test_device_copy(count):
    """gennmi_copy_f32: every element copied, nothing beyond `count` touched (odd counts take the scalar tail)."""
    from genn_amd import _abi
    from genn_amd.genn_model import Array
    _abi.check(_abi.load().gennmi_init(0))
    src, dst = Array(count + 8, np.float32), Array(count + 8, np.float32, fill=-1.0)
    src.view[:] = np.arange(count + 8, dtype=np.float32)
    src.push_to_device()
    _abi.check(_abi.load().gennmi_copy_f32(dst.ptr, src.ptr, count))
    got = dst.pull_from_device()
    assert np.array_equal(got[:count], src.view[:count])
    assert np.all(got[count:] == -1.0)
    src.free(); dst.free()


@pytest.mark.parametrize("replay", [False, True])
def test_spike_source_arrays_rewritten_between_steps(replay):
    """The neuron update keeps the time of each source's next spike beside its state instead of gathering
    spikeTimes[startSpike] every step; that copy must follow the user's arrays.  After 25 steps the host rewinds startSpike
    and shifts spikeTimes by 30 ms (the way new input is fed to a SpikeSourceArray): the same pattern must come out again,
    30 steps later, through single steps and through replayed graphs."""
    n, first = 300, 25
    rng = np.random.default_rng(12)
    per = rng.integers(0, 4, n)                                  # 0..3 spikes per source
    end = np.cumsum(per).astype(np.uint32)
    start = (end - per).astype(np.uint32)
    times = np.concatenate([np.sort(rng.choice(20, k, replace=False)) for k in per] + [np.zeros(0)]).astype(np.float32)
    model = GeNNModel("float", "rewrite", dt=1.0)
    src = model.add_neuron_population("S", n, "SpikeSourceArray", {}, {"startSpike": start, "endSpike": end})
    src.set_extra_global_param("spikeTimes", np.concatenate([times, [0.0]]))
    src.spike_recording_enabled = True
    model.build()
    model.load(num_recording_timesteps=80)

    def expected(offset):
        want = np.zeros((80, n), bool)
        for i in range(n):
            for t in times[start[i]:end[i]]:
                want[int(t) + offset, i] = True
        return want

    for _ in range(first):
        model.step_time()
    assert np.array_equal(src.vars["startSpike"].pull_from_device(), end)            # every source has used up its list
    src.vars["spikeTimes"].view[:len(times)] = times + 30.0
    src.vars["spikeTimes"].push_to_device()
    src.vars["startSpike"].view[:] = start
    src.vars["startSpike"].push_to_device()
    if replay:
        model.run(55)
    else:
        for _ in range(55):
            model.step_time()
    model.pull_recording_buffers_from_device()
    words = src.vars["recordSpk"].view.reshape(80, -1)
    got = np.unpackbits(words.view(np.uint8), axis=1, bitorder="little")[:, :n].astype(bool)
    assert np.array_equal(got, expected(0) | expected(30))
    assert got.sum() == 2 * per.sum() and per.sum() > 300
    model.unload()


def test_column_view_of_columns_longer_than_the_lds_sort():
    """gennmi_build_remap with columns beyond 16,384 entries (the reference's remap build has no limit on the column length,
    backendSIMT.cc:1977-1991): two long columns (40,000 and 20,001 entries) among short and empty ones; every column of the
    view must list its synapses in ascending idSyn — the order of the CPU backend's row-major build
    (single_threaded_cpu/backend.cc:156-179) — and the lengths must be the counts."""
    import ctypes as C
    from genn_amd import _abi
    from genn_amd.genn_model import Array
    lib = _abi.load()
    _abi.check(lib.gennmi_init(0))
    num_src, num_trg, row_stride = 40000, 7, 4
    rng = np.random.default_rng(5)
    ind = np.zeros((num_src, row_stride), np.uint32)
    row_length = np.zeros(num_src, np.uint32)
    for i in range(num_src):
        targets = [0]                                   # every row reaches column 0
        if i % 2 == 0 or i == 1:
            targets.append(3)                           # 20,001 rows reach column 3
        if i % 97 == 0:
            targets.append(5)
        if i == 12345:
            targets.append(6)
        targets.sort()
        row_length[i] = len(targets)
        ind[i, :len(targets)] = targets
        ind[i, len(targets):] = rng.integers(0, num_trg, row_stride - len(targets))       # padding: never read
    want = [[] for _ in range(num_trg)]
    for i in range(num_src):
        for j in range(row_length[i]):
            want[ind[i, j]].append(i * row_stride + j)
    col_stride = max(len(c) for c in want)
    assert col_stride == 40000 and len(want[3]) == 20001 and not want[1]
    arrays = {}
    for name, host in (("rowLength", row_length), ("ind", ind.reshape(-1))):
        a = Array(host.size, np.uint32)
        a.view[:] = host
        a.push_to_device()
        arrays[name] = a
    col_length = Array(num_trg, np.uint32, device_only=True)
    remap = Array(num_trg * col_stride, np.uint32, device_only=True)
    _abi.check(lib.gennmi_build_remap(num_src, num_trg, row_stride, col_stride, arrays["rowLength"].ptr, arrays["ind"].ptr, col_length.ptr, remap.ptr))
    got_length = col_length.pull_from_device().copy()
    got = remap.pull_from_device().reshape(num_trg, col_stride).copy()
    for a in (*arrays.values(), col_length, remap):
        a.free()
    assert np.array_equal(got_length, [len(c) for c in want])
    for j in range(num_trg):
        assert np.array_equal(got[j, :len(want[j])], np.asarray(want[j], dtype=np.uint32)), f"column {j}"
