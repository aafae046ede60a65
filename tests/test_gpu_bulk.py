"""The neuron update for large populations (four neurons per lane, all inputs requested before anything is stored),
forced onto small networks: it must leave every array exactly as the one-neuron-per-lane kernel and the CPU oracle do."""
import numpy as np
import pytest

from genn_amd import configs, rng
from genn_amd.netspec import Net, Pop, Syn
from parity import run_side_by_side

pytestmark = pytest.mark.gpu


@pytest.fixture(autouse=True)
def _bulk(monkeypatch):
    monkeypatch.setenv("GENNMI_NEURON_BULK", "1")
    monkeypatch.setenv("GENNMI_RESIDENT", "0")


@pytest.mark.parametrize("n", [1, 63, 64, 65, 255, 256, 257, 1023, 1024, 1025, 5000])
def test_ragged_population_sizes(n, monkeypatch):
    """Sizes around the chunk (64), the wave's share (256) and the work-group's share (1024); everyone fires in step 0."""
    monkeypatch.setenv("GENNMI_TILE_FLOATS", "0")
    lif = dict(C=1.0, TauM=20.0, Vrest=-60.0, Vreset=-60.0, Vthresh=-50.0, Ioffset=1.0, TauRefrac=2.0)
    net = Net(name="ragged_bulk", dt=1.0, steps=40)
    net.pops.append(Pop("A", "lif", n, dict(lif), {"V": np.full(n, -50.5, np.float32), "RefracTime": np.zeros(n, np.float32)}))
    m = max(1, n // 2)
    net.pops.append(Pop("B", "lif", m, dict(lif, Ioffset=0.2), {"V": np.full(m, -60.0, np.float32), "RefracTime": np.zeros(m, np.float32)}))
    stride = 5
    row_length = (rng.randint(3, 1, 0, n, stride + 1)).astype(np.uint32)
    ind = np.sort(rng.randint(3, 2, 0, n * stride, m).reshape(n, stride), axis=1).astype(np.uint32)
    net.syns.append(Syn("AB", "A", "B", wum="static", psm="expcurr", tau=5.0, row_stride=stride, row_length=row_length, ind=ind,
                        g=np.full((n, stride), 1.5, np.float32)))
    model, oracle, counts = run_side_by_side(net, check_every=10, exact=True)
    assert model.runner_info()["bulk_neuron_kernel"]
    assert counts["A"] >= n
    model.unload()


def test_balanced_network_two_postsynaptic_models():
    net = configs.vogels_abbott(n=4000, steps=600)
    model, oracle, counts = run_side_by_side(net, check_every=100, exact=True)
    assert model.runner_info()["bulk_neuron_kernel"]
    assert counts["E"] > 500 and counts["I"] > 100
    model.unload()


def test_many_work_groups_every_one_with_spikes():
    """70,000 uncoupled-looking neurons with staggered phases: 69 work-groups, so queue offsets cross the boundary between
    two groups of 64 whose totals are published separately, and nearly every work-group emits spikes in every step."""
    n = 70000
    lif = dict(C=1.0, TauM=20.0, Vrest=-60.0, Vreset=-60.0, Vthresh=-50.0, Ioffset=1.2, TauRefrac=1.0)
    net = Net(name="many_groups", dt=1.0, steps=40)
    net.pops.append(Pop("A", "lif", n, dict(lif), {"V": (-60.0 + 10.0 * rng.uniform(8, 1, 0, n)).astype(np.float32), "RefracTime": np.zeros(n, np.float32)}))
    net.pops.append(Pop("B", "lif", 300, dict(lif, Ioffset=0.1), {"V": np.full(300, -60.0, np.float32), "RefracTime": np.zeros(300, np.float32)}))
    ind = rng.randint(8, 2, 0, n, 300).reshape(n, 1).astype(np.uint32)
    net.syns.append(Syn("AB", "A", "B", wum="static", psm="expcurr", tau=5.0, row_stride=1, row_length=np.ones(n, np.uint32), ind=ind,
                        g=np.full((n, 1), 0.0078125, np.float32)))
    model, oracle, counts = run_side_by_side(net, check_every=10, exact=True)
    assert model.runner_info()["bulk_neuron_kernel"]
    assert counts["A"] > 3 * n
    model.unload()


def test_dendritic_delay_rings(monkeypatch):
    """Front slot of the delay ring read and cleared by the bulk kernel (microcircuit shape, fused postsynaptic models)."""
    net = configs.potjans(neuron_scale=0.05, connectivity_scale=1.0, steps=300)
    model, oracle, counts = run_side_by_side(net, check_every=50, exact=False, exact_steps=300)
    info = model.runner_info()
    assert info["bulk_neuron_kernel"] and not info["single_launch_step"]
    assert sum(counts.values()) > 100
    model.unload()


def test_izhikevich_with_noise_source():
    net = configs.izhikevich_fanout(n=6000, fanout=100, steps=150)
    model, oracle, counts = run_side_by_side(net, check_every=25, exact=False, exact_steps=60)
    assert model.runner_info()["bulk_neuron_kernel"]
    assert counts["N"] > 100
    model.unload()


def test_spike_sources_and_batches():
    """Convolution layer: spike-source chunks, LIF chunks and three batches through the bulk kernel; batch b must equal a
    batch-1 oracle run fed batch b's spike trains."""
    import copy
    from genn_amd.genn_model import model_from_net
    from oracle.genn_cpu import OracleNet
    B = 3
    nets = [configs.conv_toeplitz(h=12, w=12, ic=3, oc=5, steps=60, w_sd=0.6, batch_index=b) for b in range(B)]
    for net in nets:
        net.pop("Out").params["Ioffset"] = 0.4
    times = np.concatenate([n.pop("In").spike_times for n in nets])
    offs = np.cumsum([0] + [len(n.pop("In").spike_times) for n in nets])
    start = np.stack([n.pop("In").vars["startSpike"] + offs[b] for b, n in enumerate(nets)]).astype(np.uint32)
    end = np.stack([n.pop("In").vars["endSpike"] + offs[b] for b, n in enumerate(nets)]).astype(np.uint32)
    batched = copy.deepcopy(nets[0])
    batched.pop("In").vars = {"startSpike": start, "endSpike": end}
    batched.pop("In").spike_times = times
    model = model_from_net(batched, batch_size=B)
    model.load(num_recording_timesteps=60)
    assert model.runner_info()["bulk_neuron_kernel"]
    oracles = [OracleNet(n) for n in nets]
    total = 0
    for step in range(60):
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
