"""GPU parity: the MI355X engine against the CPU oracle on the same seeded inputs, through the C ABI.

Bars: connectivity-derived arrays (colLength/remap) and per-step spike queues bit-exact; state within
1e-5 relative — bit-exact wherever no fp32 sum can be reordered (one weight value per outPost);
rasters identical over the first 100 ms of simulated time."""
import numpy as np
import pytest

from genn_amd import configs
from genn_amd.genn_model import model_from_net
from oracle.genn_cpu import OracleNet
from parity import compare_state, run_side_by_side

pytestmark = pytest.mark.gpu


def test_balanced_lif_bit_exact():
    """C1 at full size.  One constant weight per projection and one outPost per projection: atomic
    reordering cannot change a bit, so spike queues AND all state must be identical for the run."""
    net = configs.vogels_abbott(n=4000, steps=1000)
    model, oracle, counts = run_side_by_side(net, check_every=100, exact=True)
    assert counts["E"] > 1000 and counts["I"] > 200
    model.unload()


@pytest.mark.parametrize("span", ["POSTSYNAPTIC", "PRESYNAPTIC", "WAVE"])
def test_balanced_lif_strategies(span):
    """Row-per-spike, few-lanes-per-spike and wave-per-spike mappings give identical results."""
    net = configs.vogels_abbott(n=1500, steps=300, p=0.05)
    model, oracle, counts = run_side_by_side(net, check_every=50, exact=True, span=span)
    assert counts["E"] > 100
    model.unload()


def test_microcircuit_dendritic_delay():
    """C2 shape at 5 % of the neurons with full in-degree: 8 populations, all postsynaptic models of a
    target fused into one ring buffer of 43 slots.  Weights differ, so sums may be reordered:
    rasters must be identical for the first 100 ms (1000 steps), state within 1e-5."""
    net = configs.potjans(neuron_scale=0.05, connectivity_scale=1.0, steps=1000)
    model, oracle, counts = run_side_by_side(net, check_every=100, exact=False, exact_steps=1000)
    assert model.runner_info()["single_launch_step"]
    assert sum(counts.values()) > 500
    model.unload()


def test_microcircuit_two_launch_step(monkeypatch):
    """Same network with the single-launch step switched off: synapse and neuron kernels run back to back and
    every ring slot must match the oracle, including the one read next."""
    monkeypatch.setenv("GENNMI_FUSED_STEP", "0")
    net = configs.potjans(neuron_scale=0.05, connectivity_scale=1.0, steps=300)
    model, oracle, counts = run_side_by_side(net, check_every=50, exact=False, exact_steps=300)
    assert not model.runner_info()["single_launch_step"]
    assert sum(counts.values()) > 100
    model.unload()


@pytest.mark.parametrize("tile_floats", ["8192", "600", "64"])
def test_dense_activity_tile_path(tile_floats, monkeypatch):
    """Steps that carry at least one event per target are handled by the tile kernel (LDS accumulation per tile
    of postsynaptic neurons).  Integer-valued weights and DeltaCurr input make every fp32 sum exact in any
    order, so the whole trajectory must be bit-identical to the oracle; tile sizes that do and do not divide the
    population, and multapses, are covered."""
    from genn_amd.netspec import Net, Pop, Syn
    from genn_amd import netgen
    monkeypatch.setenv("GENNMI_TILE_FLOATS", tile_floats)
    n, m, fan = 3000, 1111, 40
    lif = dict(C=1.0, TauM=20.0, Vrest=-60.0, Vreset=-60.0, Vthresh=-50.0, Ioffset=0.7, TauRefrac=2.0)
    net = Net(name="dense", dt=1.0, steps=80)
    v0 = (-60.0 + 10.0 * np.linspace(0, 1, n)).astype(np.float32)
    net.pops.append(Pop("A", "lif", n, dict(lif), {"V": v0, "RefracTime": np.zeros(n, np.float32)}))
    net.pops.append(Pop("B", "lif", m, dict(lif, Ioffset=0.0), {"V": np.full(m, -60.0, np.float32), "RefracTime": np.zeros(m, np.float32)}))
    rl, ind = netgen.fixed_number_post(11, 3, n, m, fan)
    g = np.round(netgen.rows_uniform(11, 4, rl, fan, n, 3.0, 0.0, 3.0, 0.0)).astype(np.float32) * 0.25      # multiples of 1/4 mV-ish: exact sums
    net.syns.append(Syn("AB", "A", "B", wum="static", psm="deltacurr", row_stride=fan, row_length=rl, ind=ind, g=g))
    model, oracle, counts = run_side_by_side(net, check_every=10, exact=True)
    assert counts["A"] > 2 * n and counts["B"] > m            # ~100 spikes per step x 40 targets >> 1111 targets: tile steps
    assert model.synaptic_event_count == oracle.events()
    model.unload()


@pytest.mark.parametrize("m, fan, tile_floats, records", [(4000, 100, "600", "1"), (4000, 100, "600", "0"), (1111, 40, "600", "1"), (6000, 230, "1024", "1")])
def test_tile_path_segment_records(m, fan, tile_floats, records, monkeypatch):
    """Static projections whose (row, tile) segments are short are read through segment records: one aligned record of 20
    (or 40) synapses per (row, tile), the tail of a longer segment from the row itself.  4000 targets in tiles of 600 with
    100 synapses per row: ~15 per segment, so records of 20 with overflowing segments; 1111 targets, 40 per row: ~20 per
    segment, records of 40; 6000 targets in tiles of 1024, 230 per row: ~38 per segment, records of 40 that overflow often.
    Exact sums (integer-valued weights into DeltaCurr), so everything must be bit-identical to the oracle, with and without
    the records."""
    from genn_amd.netspec import Net, Pop, Syn
    from genn_amd import netgen
    monkeypatch.setenv("GENNMI_TILE_FLOATS", tile_floats)
    monkeypatch.setenv("GENNMI_TILE_RECORDS", records)
    n = 3000
    lif = dict(C=1.0, TauM=20.0, Vrest=-60.0, Vreset=-60.0, Vthresh=-50.0, Ioffset=0.7, TauRefrac=2.0)
    net = Net(name="records", dt=1.0, steps=60)
    v0 = (-60.0 + 10.0 * np.linspace(0, 1, n)).astype(np.float32)
    net.pops.append(Pop("A", "lif", n, dict(lif), {"V": v0, "RefracTime": np.zeros(n, np.float32)}))
    net.pops.append(Pop("B", "lif", m, dict(lif, Ioffset=0.0), {"V": np.full(m, -60.0, np.float32), "RefracTime": np.zeros(m, np.float32)}))
    rl, ind = netgen.fixed_number_post(11, 3, n, m, fan)
    rl[::7] = (rl[::7] * 2) // 3            # ragged rows: the last segments of those rows are short or empty
    g = np.round(netgen.rows_uniform(11, 4, rl, fan, n, 3.0, 0.0, 3.0, 0.0)).astype(np.float32) * 0.125
    net.syns.append(Syn("AB", "A", "B", wum="static", psm="deltacurr", row_stride=fan, row_length=rl, ind=ind, g=g))
    model, oracle, counts = run_side_by_side(net, check_every=10, exact=True)
    assert counts["A"] > 2 * n
    assert model.synaptic_event_count == oracle.events()
    model.unload()


def test_izhikevich_fanout_noise():
    """C3 shape: Izhikevich neurons, fixed fanout with replacement (multapses), DeltaCurr input,
    per-step noise current from a pregenerated array.  dt = 1 ms, first 100 ms = 100 steps."""
    net = configs.izhikevich_fanout(n=20000, fanout=100, steps=200)
    model, oracle, counts = run_side_by_side(net, check_every=20, exact=False, exact_steps=100)
    assert counts["N"] > 1000
    model.unload()


@pytest.mark.parametrize("rule", ["stdp_trace", "stdp_additive"])
def test_plastic_stdp_learn_post(rule):
    """C4 shape: STDP on E->E with learnPost through the column remap, SpikeSourceArray drive — with the trace rule of the
    benchmark script and with the built-in nearest-neighbour rule (weightUpdateModels.h:345-367), whose oracle restatement
    the fixture stdp_additive_small pins to the reference's CPU backend."""
    net = configs.plastic_stdp(n=5000, n_src=100, steps=200, fan=250, src_fan=50, rule=rule)
    model = model_from_net(net)
    model.load(num_recording_timesteps=net.steps)
    sg = model.synapse_populations["EE"]
    oracle = OracleNet(net, col_stride={"EE": sg.col_stride})
    # the column view must equal the CPU build bit for bit (ascending synapse index within a column)
    col_length = sg.vars["colLength"].pull_from_device()
    assert np.array_equal(col_length, oracle.col_length("EE"))
    assert sg.col_stride == col_length.max()
    remap = sg.vars["remap"].pull_from_device().reshape(-1, sg.col_stride)
    want = oracle.remap("EE").reshape(-1, sg.col_stride)
    mask = np.arange(sg.col_stride)[None, :] < col_length[:, None]
    assert np.array_equal(remap[mask], want[mask])
    spikes = 0
    for step in range(net.steps):
        model.step_time()
        oracle.step()
        for p in net.pops:
            got = model.neuron_populations[p.name].current_spikes[0]
            want_s = oracle.spikes(p.name)
            if step < 100:
                assert np.array_equal(got, want_s), f"step {step}: spike queue of {p.name} differs"
            spikes += len(want_s)
        if step < 100 and (step + 1) % 20 == 0:
            compare_state(net, model, oracle, f"step {step}", exact=False)
    assert spikes > 2000
    model.unload()


@pytest.mark.parametrize("rule", ["stdp_trace", "stdp_additive"])
@pytest.mark.parametrize("divisor", ["1000000", "0"])
def test_learn_post_row_walk_and_column_walk(divisor, rule, monkeypatch):
    """learnPost has two device paths: columns of the spiking targets through the remap (few spikes) and a walk over
    all rows with a bitmap of the spiking targets (many spikes).  Forcing either for every step must leave the same
    weights as the oracle: each synapse gets the same single update, so g must agree to the last bit of the tolerance
    used everywhere else (and the two device paths with each other exactly)."""
    monkeypatch.setenv("GENNMI_POST_DENSE_DIVISOR", divisor)
    net = configs.plastic_stdp(n=3000, n_src=100, steps=120, fan=150, src_fan=50, rule=rule)
    model = model_from_net(net)
    model.load(num_recording_timesteps=net.steps)
    sg = model.synapse_populations["EE"]
    oracle = OracleNet(net, col_stride={"EE": sg.col_stride})
    spikes = 0
    for step in range(net.steps):
        model.step_time()
        oracle.step()
        for p in net.pops:
            want = oracle.spikes(p.name)
            assert np.array_equal(model.neuron_populations[p.name].current_spikes[0], want), f"step {step}: spike queue of {p.name} differs"
            spikes += len(want)
        if (step + 1) % 30 == 0:
            compare_state(net, model, oracle, f"step {step}", exact=False)
    assert spikes > 1000
    changed = np.count_nonzero(sg.vars["g"].pull_from_device() != net.syn("EE").g.reshape(-1))
    assert changed > 1000, "no weight was updated"
    model.unload()


def test_toeplitz_conv_layer():
    """C5 shape at 16x16x4 -> 16x16x8 (batch 1; the oracle, like the reference's CPU backend, has no batch)."""
    net = configs.conv_toeplitz(h=16, w=16, ic=4, oc=8, steps=150, w_sd=0.5)
    net.pop("Out").params["Ioffset"] = 0.4
    model, oracle, counts = run_side_by_side(net, check_every=25, exact=False, exact_steps=100)
    assert counts["Out"] > 100 and counts["In"] > 1000
    model.unload()


@pytest.mark.parametrize("h, w, ic, oc, k", [(10, 12, 3, 5, 3), (8, 40, 4, 40, 5), (6, 33, 8, 32, 5), (9, 9, 1, 3, 3)])
def test_toeplitz_conv_on_matrix_cores(h, w, ic, oc, k, monkeypatch):
    """The dense path of a Conv2D projection (fp32 MFMA over the spike bitmap) on shapes that exercise its edges: an odd
    number of input channels (a pair of sum steps straddles two kernel taps) and an odd K (zero padding row), output
    channels and widths that are no multiple of the 32 x 32 tile or need several tiles, and 5 x 5 kernels whose sum is
    longer than one unrolled chunk of steps.  Activity is high enough that every step takes the dense path; rasters must be
    the oracle's, state within 1e-5, and the event count exact."""
    net = configs.conv_toeplitz(h=h, w=w, ic=ic, oc=oc, k=k, steps=60, w_sd=0.5 / k, max_rate=400.0, ioffset=0.3)
    model, oracle, counts = run_side_by_side(net, check_every=20, exact=False, exact_steps=60)
    assert counts["Out"] > 50 and counts["In"] > 5 * h * w * ic
    assert model.synaptic_event_count == oracle.events()
    assert model.runner_info()["conv_on_matrix_cores"]
    # The whole step is one launch (postsynaptic and neuron model applied to the layer's accumulators) where a work-group's
    # neurons start on a word of the recording bitmap: two of the four shapes, one of them with 40 output channels, so that
    # a pixel's channels straddle the words of the work-group's spike bitmap.
    one_launch = model.runner_info()["conv_step_in_one_launch"]
    assert one_launch == ((w * oc) % 32 == 0)
    # the same network with the layer's kernel and the neuron kernel launched one after the other, and on the event-driven
    # kernels: same rasters, same event count
    for switch, flag in (("GENNMI_CONV_STEP", "conv_step_in_one_launch"), ("GENNMI_CONV_MFMA", "conv_on_matrix_cores")):
        monkeypatch.setenv(switch, "0")
        other = model_from_net(net)
        other.load(num_recording_timesteps=60)
        assert not other.runner_info()[flag]
        other.run(60)
        other.synchronize()
        assert other.synaptic_event_count == model.synaptic_event_count
        for p in net.pops:
            assert np.array_equal(other.neuron_populations[p.name].current_spikes[0], model.neuron_populations[p.name].current_spikes[0])
        model.pull_recording_buffers_from_device(); other.pull_recording_buffers_from_device()
        for p in net.pops:
            assert np.array_equal(other.neuron_populations[p.name].vars["recordSpk"].view, model.neuron_populations[p.name].vars["recordSpk"].view), p.name
        other.unload()
    model.unload()


def test_toeplitz_batches_are_independent():
    """Batch b of a batched run equals a batch-1 run of the oracle fed batch b's spike trains."""
    B = 3
    nets = [configs.conv_toeplitz(h=8, w=8, ic=2, oc=4, steps=60, w_sd=0.6, batch_index=b) for b in range(B)]
    for net in nets:
        net.pop("Out").params["Ioffset"] = 0.4
    base = nets[0]
    # spikeTimes is shared by all batches; startSpike / endSpike select each batch's slice (test_recording.py:56-103)
    times = np.concatenate([n.pop("In").spike_times for n in nets])
    offs = np.cumsum([0] + [len(n.pop("In").spike_times) for n in nets])
    start = np.stack([n.pop("In").vars["startSpike"] + offs[b] for b, n in enumerate(nets)]).astype(np.uint32)
    end = np.stack([n.pop("In").vars["endSpike"] + offs[b] for b, n in enumerate(nets)]).astype(np.uint32)
    import copy
    batched = copy.deepcopy(base)
    batched.pop("In").vars = {"startSpike": start, "endSpike": end}
    batched.pop("In").spike_times = times
    model = model_from_net(batched, batch_size=B)
    model.load(num_recording_timesteps=base.steps)
    oracles = [OracleNet(n) for n in nets]
    total = 0
    for step in range(base.steps):
        model.step_time()
        got = {name: model.neuron_populations[name].current_spikes for name in ("In", "Out")}
        for b, o in enumerate(oracles):
            o.step()
            for name in ("In", "Out"):
                assert np.array_equal(got[name][b], o.spikes(name)), f"step {step} batch {b}: {name} spikes differ"
                total += len(o.spikes(name))
    assert total > 500
    v = model.neuron_populations["Out"].vars["V"].pull_from_device().reshape(B, -1)
    for b, o in enumerate(oracles):
        np.testing.assert_allclose(v[b], o.var("Out", 0), rtol=1e-5)
    model.unload()


@pytest.mark.parametrize("rule, combined", [("stdp_trace", "1"), ("stdp_additive", "1"), ("stdp_trace", "0")])
def test_plastic_batches_are_independent(rule, combined, monkeypatch):
    """Batch b of a batched plastic network equals a batch-1 run of the oracle on batch b's inputs: weights a learning rule
    writes, traces and spike times are per batch (models.h: VarAccess::READ_WRITE has the batch dimension), connectivity is
    shared.  The batches differ in their initial membrane potentials and in their Poisson spike trains.  Run with the
    scatter / tile / learnPost passes sharing one launch and with a launch each."""
    monkeypatch.setenv("GENNMI_COMBINED", combined)
    import copy
    from genn_amd import rng
    from genn_amd.configs import poisson_spike_source
    B, steps = 3, 120
    nets = []
    for b in range(B):
        net = configs.plastic_stdp(n=1500, n_src=100, steps=steps, fan=80, src_fan=60, rule=rule)
        if b:
            for k, name in enumerate(("E", "I")):
                p = net.pop(name)
                p.vars["V"] = (-60.0 + 10.0 * rng.uniform(1234 + b, 1 + k, 0, p.n)).astype(np.float32)
            start, end, times = poisson_spike_source(net.seed, 50 + b, 100, 10.0, steps, net.dt)
            src = net.pop("P")
            src.vars = {"startSpike": start, "endSpike": end}
            src.spike_times = times
        nets.append(net)
    batched = copy.deepcopy(nets[0])
    for name in ("E", "I"):
        batched.pop(name).vars = {"V": np.stack([n.pop(name).vars["V"] for n in nets]), "RefracTime": np.zeros((B, nets[0].pop(name).n), np.float32)}
    offs = np.cumsum([0] + [len(n.pop("P").spike_times) for n in nets])
    batched.pop("P").vars = {"startSpike": np.stack([n.pop("P").vars["startSpike"] + offs[b] for b, n in enumerate(nets)]).astype(np.uint32),
                             "endSpike": np.stack([n.pop("P").vars["endSpike"] + offs[b] for b, n in enumerate(nets)]).astype(np.uint32)}
    batched.pop("P").spike_times = np.concatenate([n.pop("P").spike_times for n in nets])
    model = model_from_net(batched, batch_size=B)
    model.load(num_recording_timesteps=steps)
    info = model.runner_info()
    assert info["combined_synapse_launch"] == (combined == "1") and info["postsynaptic_in_combined_launch"] == (combined == "1")
    oracles = [OracleNet(n) for n in nets]
    total = 0
    for step in range(steps):
        model.step_time()
        got = {p.name: model.neuron_populations[p.name].current_spikes for p in batched.pops}
        for b, o in enumerate(oracles):
            o.step()
            for p in batched.pops:
                assert np.array_equal(got[p.name][b], o.spikes(p.name)), f"step {step} batch {b}: {p.name} spikes differ"
                total += len(o.spikes(p.name))
    assert total > 1500
    g = model.synapse_populations["EE"].vars["g"].pull_from_device().reshape(B, -1)
    v = model.neuron_populations["E"].vars["V"].pull_from_device().reshape(B, -1)
    for b, o in enumerate(oracles):
        # every weight has one writer per step and the rules are evaluated as the oracle evaluates them: identical
        assert np.array_equal(g[b], o.syn_g("EE").reshape(-1)), f"batch {b}: weights differ"
        np.testing.assert_allclose(v[b], o.var("E", 0), rtol=1e-5, atol=1e-5)
        assert np.count_nonzero(g[b] != nets[b].syn("EE").g.reshape(-1)) > 500
    assert not np.array_equal(g[0], g[1])
    model.unload()


@pytest.mark.parametrize("span", ["POSTSYNAPTIC", "PRESYNAPTIC"])
def test_axonal_delays(span):
    """Balanced LIF network with axonal delays of 3, 1, 0 and 5 timesteps: the spike queue of a population is a ring of
    slots (4 for E, 6 for I) and every projection reads the slot its delay selects.  One weight per outPost, so the whole
    state must be identical to the oracle's, stepped one launch at a time and through graph replay."""
    delays = {"EE": 3, "EI": 1, "IE": 0, "II": 5}
    net = configs.vogels_abbott(n=2000, steps=600, p=0.04, axonal_delays=delays)
    model, oracle, counts = run_side_by_side(net, check_every=100, exact=True, span=span)
    assert counts["E"] > 300 and counts["I"] > 50
    info = model.runner_info()
    assert not info["resident_plan"] and not info["single_launch_step"]
    # the same network through run(): graph replays of the two-launch step
    replay = model_from_net(net, span=span)
    replay.load(num_recording_timesteps=600)
    replay.run(600)
    replay.synchronize()
    for p in net.pops:
        for name in ("V", "RefracTime"):
            assert np.array_equal(replay.neuron_populations[p.name].vars[name].pull_from_device(), model.neuron_populations[p.name].vars[name].pull_from_device())
        assert np.array_equal(replay.neuron_populations[p.name].current_spikes[0], oracle.spikes(p.name))
    assert replay.synaptic_event_count == model.synaptic_event_count == oracle.events()
    replay.unload()
    model.unload()


@pytest.mark.parametrize("fuse", [False, True])
def test_dense_and_bitmask_projections(fuse):
    """DENSE (individual and constant weights), BITMASK and constant-weight SPARSE projections in a recurrent LIF network
    whose populations are not multiples of the wavefront or of a connectivity word.  A lane that owns its outPost
    element continues the sum in spike-queue order, the CPU backend's order, so without fusing everything is identical;
    with fused postsynaptic models several projections share an outPost (partial sums, one atomic each) and state is
    held to 1e-5."""
    net = configs.dense_bitmask(fuse=fuse)
    model, oracle, counts = run_side_by_side(net, check_every=20, exact=not fuse, exact_steps=100)
    assert counts["A"] > 1000 and counts["B"] > 50
    assert model.synaptic_event_count == oracle.events()
    model.unload()


def test_dense_layer_many_spikes_per_step():
    """A DENSE layer in which a step carries hundreds of spikes: the queue is cut into pieces handled by different blocks,
    each adding a partial sum.  Weights are multiples of 2^-10 and the postsynaptic model keeps nothing between steps, so
    every sum is exact in any order and state, spikes and event counts must still be identical."""
    net = configs.dense_layer(n_in=2100, n_out=530, rate_hz=120.0, steps=60, w_sd=0.03)
    syn = net.syns[0]
    syn.g = (np.rint(syn.g * 1024.0) / 1024.0).astype(np.float32)
    syn.psm = "deltacurr"
    model, oracle, counts = run_side_by_side(net, check_every=10, exact=True)
    assert counts["In"] > 60 * 200 and counts["Out"] > 50
    assert model.synaptic_event_count == oracle.events() == (counts["In"] - len(oracle.spikes("In"))) * 530
    model.unload()


def test_dense_projection_batched():
    """Batch of 3 through a DENSE projection: weights are shared, spike queues and outPost are per batch."""
    from genn_amd.genn_model import GeNNModel, init_postsynaptic, init_weight_update
    B, n_src, n_trg = 3, 40, 70
    model = GeNNModel("float", "dense_batch", batch_size=B, dt=1.0)
    start = np.stack([np.arange(n_src), np.arange(n_src), np.arange(n_src)]).astype(np.uint32)
    # batch b's source i fires at step (i + b) % 7
    times = np.stack([(np.arange(n_src) + b) % 7 for b in range(B)]).astype(np.float32)
    src = model.add_neuron_population("S", n_src, "SpikeSourceArray", {}, {"startSpike": start + np.arange(B)[:, None] * n_src,
                                                                          "endSpike": start + np.arange(B)[:, None] * n_src + 1})
    src.set_extra_global_param("spikeTimes", times.reshape(-1))
    lif = {"C": 1.0, "TauM": 20.0, "Vrest": -60.0, "Vreset": -60.0, "Vthresh": 1e9, "Ioffset": 0.0, "TauRefrac": 5.0}
    trg = model.add_neuron_population("T", n_trg, "LIF", lif, {"V": -60.0, "RefracTime": 0.0})
    w = np.arange(n_src * n_trg, dtype=np.float32).reshape(n_src, n_trg) % 13 - 6
    s = model.add_synapse_population("ST", "DENSE", src, trg, init_weight_update("StaticPulse", {}, {"g": w.flatten()}), init_postsynaptic("DeltaCurr"))
    model.build()
    model.load()
    for step in range(9):
        model.update_synapses()
        got = s.vars["outPost"].pull_from_device().reshape(B, n_trg)
        for b in range(B):
            fired = (times[b] == step - 1) if step > 0 else np.zeros(n_src, bool)
            assert np.array_equal(got[b], w.T @ fired.astype(np.float32)), f"step {step}, batch {b}"
        model.update_neurons()
    model.unload()


@pytest.mark.parametrize("resident", ["1", "0"])
def test_graph_replay_matches_stepping(resident, monkeypatch):
    """run() either keeps the network resident on the chip for the whole chunk (one launch) or, with that plan switched
    off, replays captured HIP graphs; either way every chunk must leave the state eager stepping leaves.
    Chunks are interleaved with eager steps and synchronisations."""
    monkeypatch.setenv("GENNMI_RESIDENT", resident)
    net = configs.vogels_abbott(n=2000, steps=730, p=0.04)
    eager = model_from_net(net)
    eager.load(num_recording_timesteps=net.steps)
    graph = model_from_net(net)
    graph.load(num_recording_timesteps=net.steps)
    assert graph.runner_info()["resident_plan"] == (resident == "1")
    for chunk in (250, 3, 200, 77, 200):           # 200/250 -> graph replays (+ remainder), 3/77 -> single steps
        graph.run(chunk)
        graph.synchronize()
        for _ in range(chunk):
            eager.step_time()
        eager.synchronize()
        for name in ("E", "I"):
            for var in ("V", "RefracTime"):
                assert np.array_equal(graph.neuron_populations[name].vars[var].pull_from_device(),
                                      eager.neuron_populations[name].vars[var].pull_from_device()), f"{name}.{var} after {graph.timestep} steps"
            assert np.array_equal(graph.neuron_populations[name].current_spikes[0], eager.neuron_populations[name].current_spikes[0])
    assert graph.timestep == eager.timestep == 730
    graph.pull_recording_buffers_from_device()
    eager.pull_recording_buffers_from_device()
    for name in ("E", "I"):
        assert np.array_equal(graph.neuron_populations[name].vars["recordSpk"].view, eager.neuron_populations[name].vars["recordSpk"].view)
    t, ids = graph.neuron_populations["E"].spike_recording_data[0]
    assert len(ids) > 500
    assert graph.synaptic_event_count == eager.synaptic_event_count
    graph.unload()
    eager.unload()


@pytest.mark.parametrize("resident", ["1", "0"])
def test_graph_replay_single_launch_step(resident, monkeypatch):
    """Chunks of steps of a dendritic-delay network — resident plan, or graph replay of the one-launch-per-step plan —
    against eager stepping (one launch per step, which hands front-slot synapses over one step early) and the oracle:
    rasters identical, membrane potentials within tolerance (weights differ, so the order of additions may differ)."""
    monkeypatch.setenv("GENNMI_RESIDENT", resident)
    net = configs.potjans(neuron_scale=0.04, connectivity_scale=1.0, steps=450)
    eager = model_from_net(net)
    eager.load(num_recording_timesteps=net.steps)
    graph = model_from_net(net)
    graph.load(num_recording_timesteps=net.steps)
    assert graph.runner_info()["single_launch_step"] and graph.runner_info()["resident_plan"] == (resident == "1")
    oracle = OracleNet(net, num_recording_timesteps=net.steps)
    for chunk in (200, 50, 200):
        graph.run(chunk)
        graph.synchronize()
        for _ in range(chunk):
            eager.step_time()
        oracle.run(chunk)
        for p in net.pops:
            want = oracle.var(p.name, 0)
            for m in (graph, eager):
                np.testing.assert_allclose(m.neuron_populations[p.name].vars["V"].pull_from_device(), want, rtol=1e-5)
    graph.pull_recording_buffers_from_device()
    eager.pull_recording_buffers_from_device()
    spikes = 0
    for p in net.pops:
        want = oracle.record(p.name, net.steps)
        assert np.array_equal(graph.neuron_populations[p.name].vars["recordSpk"].view, want)
        assert np.array_equal(eager.neuron_populations[p.name].vars["recordSpk"].view, want)
        spikes += int(np.unpackbits(want.view(np.uint8)).sum())
    assert spikes > 200
    assert graph.synaptic_event_count == eager.synaptic_event_count == oracle.events()
    graph.unload()
    eager.unload()


@pytest.mark.parametrize("n", [1, 31, 64, 65, 257, 1000])
def test_ragged_population_sizes(n, monkeypatch):
    """Population sizes around the wave (64), recording-word (32) and work-group (256) boundaries;
    includes empty rows and a population in which every neuron fires in the same step.  The tile path is
    switched off: it adds LDS partial sums to outPost, which re-associates the sum (tested separately)."""
    monkeypatch.setenv("GENNMI_TILE_FLOATS", "0")
    from genn_amd.netspec import Net, Pop, Syn
    from genn_amd import rng
    lif = dict(C=1.0, TauM=20.0, Vrest=-60.0, Vreset=-60.0, Vthresh=-50.0, Ioffset=1.0, TauRefrac=2.0)
    net = Net(name="ragged", dt=1.0, steps=60)
    v0 = np.full(n, -50.5, np.float32)             # everyone crosses threshold in step 0
    net.pops.append(Pop("A", "lif", n, dict(lif), {"V": v0, "RefracTime": np.zeros(n, np.float32)}))
    m = max(1, n // 2)
    net.pops.append(Pop("B", "lif", m, dict(lif, Ioffset=0.2), {"V": np.full(m, -60.0, np.float32), "RefracTime": np.zeros(m, np.float32)}))
    stride = 5
    row_length = (rng.randint(3, 1, 0, n, stride + 1)).astype(np.uint32)      # 0..5, some rows empty
    ind = np.sort(rng.randint(3, 2, 0, n * stride, m).reshape(n, stride), axis=1).astype(np.uint32)
    g = np.full((n, stride), 1.5, np.float32)
    net.syns.append(Syn("AB", "A", "B", wum="static", psm="expcurr", tau=5.0, row_stride=stride, row_length=row_length, ind=ind, g=g))
    model, oracle, counts = run_side_by_side(net, check_every=10, exact=True)
    assert counts["A"] >= n
    model.unload()
