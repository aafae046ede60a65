"""Connectivity written after load (pygenn's push_connectivity_to_device in the middle of a run): the tables the runner
derives from rowLength / ind / d — segment boundaries of the tile path, zero-delay lists of the single-launch step, column
views of ordered accumulation, the resident plan's segment tables — must follow it."""
import numpy as np
import pytest

from genn_amd import configs, netgen
from genn_amd.genn_model import model_from_net
from genn_amd.netspec import Net, Pop, Syn
from oracle.genn_cpu import OracleNet
from parity import compare_state

pytestmark = pytest.mark.gpu


def _exact_net():
    """Integer-valued weights into DeltaCurr input: every fp32 sum is exact in any order."""
    n, m, fan = 3000, 1111, 40
    lif = dict(C=1.0, TauM=20.0, Vrest=-60.0, Vreset=-60.0, Vthresh=-50.0, Ioffset=0.7, TauRefrac=2.0)
    net = Net(name="push", dt=1.0, steps=80)
    v0 = (-60.0 + 10.0 * np.linspace(0, 1, n)).astype(np.float32)
    net.pops.append(Pop("A", "lif", n, dict(lif), {"V": v0, "RefracTime": np.zeros(n, np.float32)}))
    net.pops.append(Pop("B", "lif", m, dict(lif, Ioffset=0.0), {"V": np.full(m, -60.0, np.float32), "RefracTime": np.zeros(m, np.float32)}))
    rl, ind = netgen.fixed_number_post(11, 3, n, m, fan)
    g = np.round(netgen.rows_uniform(11, 4, rl, fan, n, 3.0, 0.0, 3.0, 0.0)).astype(np.float32) * 0.25
    net.syns.append(Syn("AB", "A", "B", wum="static", psm="deltacurr", row_stride=fan, row_length=rl, ind=ind, g=g))
    return net


@pytest.mark.parametrize("ordered", [False, True])
def test_rewritten_rows_on_the_tile_path(ordered):
    net = _exact_net()
    syn = net.syns[0]
    model = model_from_net(net, ordered=ordered)
    model.load(num_recording_timesteps=net.steps)
    oracle = OracleNet(net, num_recording_timesteps=net.steps)

    def both(steps):
        for _ in range(steps):
            model.step_time()
            oracle.step()
            for p in net.pops:
                assert np.array_equal(model.neuron_populations[p.name].current_spikes[0], oracle.spikes(p.name)), f"step {model.timestep}: {p.name}"

    both(25)
    # half of the rows get new targets (sorted, like the old ones) and a different length; the oracle reads the same arrays
    m = net.pop("B").n
    rows = np.arange(0, net.pop("A").n, 2)
    syn.ind[rows] = np.sort((syn.ind[rows].astype(np.int64) * 7 + 13) % m, axis=1).astype(np.uint32)
    syn.row_length[rows] = (syn.row_length[rows] * 3) // 4
    sg = model.synapse_populations["AB"]
    sg.vars["ind"].view[:] = syn.ind.reshape(-1)
    sg.vars["rowLength"].view[:] = syn.row_length
    sg.vars["ind"].push_to_device()
    sg.vars["rowLength"].push_to_device()
    both(40)
    compare_state(net, model, oracle, "after the push", exact=True)
    assert model.synaptic_event_count == oracle.events()
    model.unload()


def test_rewritten_weights_reach_the_segment_records(monkeypatch):
    """The tile path's segment records hold copies of the weights: a weight push in the middle of a run must reach them."""
    monkeypatch.setenv("GENNMI_TILE_FLOATS", "600")
    net = _exact_net()                      # 1111 targets in tiles of 600, 40 synapses per row: records of 40
    syn = net.syns[0]
    model = model_from_net(net)
    model.load(num_recording_timesteps=net.steps)
    oracle = OracleNet(net, num_recording_timesteps=net.steps)
    for phase in range(2):
        for _ in range(30):
            model.step_time()
            oracle.step()
            for p in net.pops:
                assert np.array_equal(model.neuron_populations[p.name].current_spikes[0], oracle.spikes(p.name)), f"step {model.timestep}: {p.name}"
        if phase == 0:
            syn.g[:] = (syn.g * 0.5 + 0.25).astype(np.float32)          # still multiples of 1/8: sums stay exact
            sg = model.synapse_populations["AB"]
            sg.vars["g"].view[:] = syn.g.reshape(-1)
            sg.vars["g"].push_to_device()
    compare_state(net, model, oracle, "after the weight push", exact=True)
    assert model.synaptic_event_count == oracle.events()
    model.unload()


@pytest.mark.parametrize("ordered", [False, True])
def test_rewritten_delays(ordered):
    """Delays of six projections are set to zero for half of their rows in the middle of a run.  Default mode: the network is
    on the single-launch step, where those synapses join the zero-delay lists (delivered by the spiking neuron's own
    wavefront) — the lists must be rebuilt, and the resident plan's segment tables with them; rasters must stay identical to
    the oracle's while reassociated sums allow (checked for 150 steps after the push; this network parts from the oracle
    near step 343 in every default plan).  Ordered accumulation: the column views are rebuilt and the captured step graph,
    which holds their addresses, is captured again; there the whole run must be identical bit for bit."""
    net = configs.potjans(neuron_scale=0.05, connectivity_scale=1.0, steps=400)
    model = model_from_net(net, ordered=ordered)
    model.load(num_recording_timesteps=400)
    assert model.runner_info()["single_launch_step"] == (not ordered)
    oracle = OracleNet(net, num_recording_timesteps=400)
    model.run(100)
    oracle.run(100)
    for s in net.syns[:6]:
        s.d[0:s.d.shape[0] // 2] = 0
        sg = model.synapse_populations[s.name]
        sg.vars["d"].view[:] = s.d.reshape(-1)
        sg.vars["d"].push_to_device()
    for _ in range(50):
        model.step_time()
        oracle.step()
        for p in net.pops:
            assert np.array_equal(model.neuron_populations[p.name].current_spikes[0], oracle.spikes(p.name)), f"step {model.timestep}: {p.name}"
    compare_state(net, model, oracle, "50 steps after the push", exact=ordered)
    model.run(250)
    oracle.run(250)
    model.pull_recording_buffers_from_device()
    identical = 400 if ordered else 250
    for p in net.pops:
        words = (p.n + 31) // 32
        got = model.neuron_populations[p.name].vars["recordSpk"].view.reshape(400, words)[:identical]
        want = oracle.record(p.name, 400).reshape(400, words)[:identical]
        assert np.array_equal(got, want), p.name
    if ordered:
        compare_state(net, model, oracle, "after 400 steps", exact=True)
    model.unload()
