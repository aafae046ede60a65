"""The resident plan (many timesteps per launch; neuron state in registers, delay rings in LDS, tiles exchanging their
spikes through one word each) against the CPU oracle, on the paths the benchmark networks do not reach often:
segments with more due synapses than an entry holds inline, steps with more (spike, projection) pairs than a tile
stages at once, tiles with many spikes in one step (side buffer), weights pushed between launches.

Weights are one value per projection and every postsynaptic model has one incoming projection, so no fp32 sum depends
on the order of its additions and everything — state, rings, spike queues, recordings, event counts — must be identical.
"""
import numpy as np
import pytest

from genn_amd import rng
from genn_amd.genn_model import model_from_net
from genn_amd.netspec import Net, Pop, Syn
from oracle.genn_cpu import OracleNet
from parity import compare_state

pytestmark = pytest.mark.gpu

LIF = dict(C=1.0, TauM=20.0, Vrest=-60.0, Vreset=-60.0, Vthresh=-50.0, Ioffset=0.0, TauRefrac=2.0)


def _pop(name, n, ioffset, v0):
    return Pop(name, "lif", n, dict(LIF, Ioffset=ioffset), {"V": np.asarray(v0, np.float32), "RefracTime": np.zeros(n, np.float32)})


def _projection(name, src, trg, n_src, n_trg, stride, weight, seed, depth=0, due_share=0.0, tau=5.0):
    """Random ascending rows of exactly `stride` targets; with depth > 0 a dendritic delay per synapse, a share
    `due_share` of which is a multiple of the ring depth (those land in the slot read in the step that delivers them)."""
    ind = np.sort(rng.randint(seed, 1, 0, n_src * stride, n_trg).reshape(n_src, stride), axis=1).astype(np.uint32)
    syn = Syn(name, src, trg, wum="static_delay" if depth else "static", psm="expcurr", tau=tau, row_stride=stride,
              row_length=np.full(n_src, stride, np.uint32), ind=ind, g=np.full((n_src, stride), weight, np.float32))
    if depth:
        u = rng.uniform(seed, 2, 0, n_src * stride).reshape(n_src, stride)
        later = 1 + rng.randint(seed, 3, 0, n_src * stride, depth - 1).reshape(n_src, stride)
        syn.d = np.where(u < due_share, 0, later).astype(np.uint8)
        syn.max_den_delay = depth
    return syn


def _run_chunks(net, chunks, check, resident=True):
    model = model_from_net(net)
    steps = sum(chunks)
    model.load(num_recording_timesteps=steps)
    assert model.runner_info()["resident_plan"] == resident
    oracle = OracleNet(net, num_recording_timesteps=steps)
    for chunk in chunks:
        if chunk < 0:                       # eager single steps in between
            for _ in range(-chunk):
                model.step_time()
            oracle.run(-chunk)
        else:
            model.run(chunk)
            oracle.run(chunk)
        model.synchronize()
        check(model, oracle)
    model.pull_recording_buffers_from_device()
    spikes = 0
    for p in net.pops:
        want = oracle.record(p.name, steps)
        assert np.array_equal(model.neuron_populations[p.name].vars["recordSpk"].view, want), f"recording of {p.name} differs"
        assert np.array_equal(model.neuron_populations[p.name].current_spikes[0], oracle.spikes(p.name))
        spikes += int(np.unpackbits(want.view(np.uint8)).sum())
    assert model.synaptic_event_count == oracle.events()
    return model, oracle, spikes


@pytest.mark.parametrize("due_share", [0.5, 0.04, 1.0])
def test_due_synapses_inline_and_row_walk(due_share):
    """Delayed projections between two populations of 700 and 300 neurons (3 + 2 tiles, ragged last tiles).  With half of
    the delays a multiple of the ring depth nearly every segment has more due synapses than fit inline (row walk before
    the update); with 4 % most have none or a few (inline); with all of them due nothing is left for later."""
    n_a, n_b, depth = 700, 300, 7
    net = Net(name="resident_due", dt=1.0, steps=0)
    net.pops.append(_pop("A", n_a, 0.62, -60.0 + 9.5 * rng.uniform(5, 1, 0, n_a)))
    net.pops.append(_pop("B", n_b, 0.45, -60.0 + 9.5 * rng.uniform(5, 2, 0, n_b)))
    net.syns.append(_projection("AB", "A", "B", n_a, n_b, 40, 0.11, 11, depth, due_share))
    net.syns.append(_projection("BA", "B", "A", n_b, n_a, 64, -0.07, 12, depth, due_share))
    net.syns.append(_projection("AA", "A", "A", n_a, n_a, 24, 0.05, 13, depth, due_share, tau=9.0))
    net.steps = 260

    def check(model, oracle):
        compare_state(net, model, oracle, f"after {model.timestep} steps", exact=True)

    # launches of 100, 5 and 60 steps with eager single steps (the one-launch-per-step plan) in between
    model, oracle, spikes = _run_chunks(net, (100, -3, 5, -2, 60, 90), check)
    assert model.runner_info()["single_launch_step"]
    assert spikes > 2000
    model.unload()


@pytest.mark.parametrize("depth", [0, 5])
def test_more_pairs_than_a_tile_stages(depth):
    """3,000 neurons cross threshold in the same step: every tile of the target sees 3,000 (spike, projection) pairs in one
    exchange, more than it stages at once, and every source tile sends 256 spikes through the side buffer."""
    n_a, n_b = 3000, 520
    net = Net(name="resident_burst", dt=1.0, steps=0)
    net.pops.append(_pop("A", n_a, 1.0, np.full(n_a, -50.4)))
    net.pops.append(_pop("B", n_b, 0.3, np.full(n_b, -58.0)))
    net.syns.append(_projection("AB", "A", "B", n_a, n_b, 12, 0.002, 21, depth, 0.3))
    net.syns.append(_projection("BA", "B", "A", n_b, n_a, 30, -0.05, 22, depth, 0.3))
    net.steps = 80

    def check(model, oracle):
        compare_state(net, model, oracle, f"after {model.timestep} steps", exact=True)

    model, oracle, spikes = _run_chunks(net, (6, 34, 40), check)
    first = oracle.record("A", 80).reshape(80, -1)[0]
    assert int(np.unpackbits(first.view(np.uint8)).sum()) == n_a          # the burst happened in step 0
    assert spikes > 2 * n_a
    model.unload()


@pytest.mark.parametrize("n_a, ioffset", [(400, 1.0), (24, 0.62), (12, 0.62)])
def test_long_row_parts_take_several_trips(n_a, ioffset):
    """Rows of 120 targets inside one tile of 200 neurons: a pair's part is longer than what its group of lanes reads in
    one trip to memory when many pairs are staged (400 sources crossing threshold together: 4 lanes per pair, 32 synapses
    per trip), and fits one trip when few are (24 or 12 sources firing now and then: 8 or 16 lanes per pair)."""
    n_b, depth = 200, 6
    net = Net(name="resident_long_parts", dt=1.0, steps=0)
    v0 = np.full(n_a, -50.4) if n_a == 400 else -60.0 + 9.5 * rng.uniform(41, 1, 0, n_a)
    net.pops.append(_pop("A", n_a, ioffset, v0))
    net.pops.append(_pop("B", n_b, 0.3, np.full(n_b, -58.0)))
    net.syns.append(_projection("AB", "A", "B", n_a, n_b, 120, 0.004 if n_a == 400 else 0.05, 42, depth, 0.1))
    net.steps = 90

    def check(model, oracle):
        compare_state(net, model, oracle, f"after {model.timestep} steps", exact=True)

    model, oracle, spikes = _run_chunks(net, (30, 60), check)
    assert spikes > (n_a if n_a == 400 else 20)
    model.unload()


def test_pushed_weights_reach_the_inline_copies(monkeypatch):
    """The segment tables hold copies of the weights of due synapses; a push of `g` between launches must refresh them.
    (With the one-launch-per-step plan the due synapses of the last step's spikes are already in the ring when the push
    happens — at their old weights, where the reference would add them after the push — so that plan is switched off
    here: the test is about the copies.)"""
    monkeypatch.setenv("GENNMI_FUSED_STEP", "0")
    n, depth = 600, 4
    net = Net(name="resident_push", dt=1.0, steps=0)
    net.pops.append(_pop("A", n, 0.6, -60.0 + 9.5 * rng.uniform(7, 1, 0, n)))
    net.syns.append(_projection("AA", "A", "A", n, n, 48, 0.04, 31, depth, 0.4))
    net.steps = 120

    state = {"pushed": False}

    def check(model, oracle):
        compare_state(net, model, oracle, f"after {model.timestep} steps", exact=True)
        if not state["pushed"]:
            g = model.synapse_populations["AA"].vars["g"]
            g.view[:] = np.float32(-0.03)
            g.push_to_device()
            oracle.syn_g("AA")[:] = np.float32(-0.03)
            state["pushed"] = True

    model, oracle, spikes = _run_chunks(net, (60, 60), check)
    assert spikes > 500
    model.unload()


def test_weights_written_behind_the_library_are_reported(monkeypatch):
    """A caller that overwrites `g` by its own means (here: a device-to-device copy the runner is not told about) and then
    names the range with gennmi_note_device_write gets the same refresh of the inline copies and packed records as a push."""
    import ctypes as C
    from genn_amd import _abi
    monkeypatch.setenv("GENNMI_FUSED_STEP", "0")
    n, depth = 600, 4
    net = Net(name="resident_note", dt=1.0, steps=0)
    net.pops.append(_pop("A", n, 0.6, -60.0 + 9.5 * rng.uniform(7, 1, 0, n)))
    net.syns.append(_projection("AA", "A", "A", n, n, 48, 0.04, 31, depth, 0.4))
    net.steps = 120
    state = {"written": False}

    def check(model, oracle):
        compare_state(net, model, oracle, f"after {model.timestep} steps", exact=True)
        if not state["written"]:
            g = model.synapse_populations["AA"].vars["g"]
            lib = _abi.load()
            staging = C.c_void_p()
            _abi.check(lib.gennmi_malloc(C.byref(staging), g.view.nbytes))
            new = np.full(g.count, -0.03, np.float32)
            _abi.check(lib.gennmi_memcpy_to_device(staging, new.ctypes.data_as(C.c_void_p), new.nbytes))
            hip = C.CDLL("libamdhip64.so")
            assert hip.hipMemcpy(C.c_void_p(g.ptr), staging, C.c_size_t(new.nbytes), C.c_int(3)) == 0      # hipMemcpyDeviceToDevice
            _abi.check(lib.gennmi_note_device_write(C.c_void_p(g.ptr), new.nbytes))
            lib.gennmi_free(staging)
            oracle.syn_g("AA")[:] = np.float32(-0.03)
            state["written"] = True

    model, oracle, spikes = _run_chunks(net, (60, 60), check)
    assert spikes > 500
    model.unload()


def test_writes_named_through_a_registered_host_buffer(monkeypatch):
    """The same for callers that only know host pointers (generated custom update code beside the library's kernels): the
    device buffer is registered behind a host buffer, gennmi_flush runs queued steps before the caller's own device work, and
    gennmi_note_mirror_write names the whole device buffer through any pointer into the host one.  One of two projections is
    rewritten: only its copies are rebuilt, and the other one's stay valid."""
    import ctypes as C
    from genn_amd import _abi
    monkeypatch.setenv("GENNMI_FUSED_STEP", "0")
    n, depth = 600, 4
    net = Net(name="resident_mirror", dt=1.0, steps=0)
    net.pops.append(_pop("A", n, 0.6, -60.0 + 9.5 * rng.uniform(17, 1, 0, n)))
    net.syns.append(_projection("AA", "A", "A", n, n, 48, 0.04, 31, depth, 0.4))
    net.syns.append(_projection("AA2", "A", "A", n, n, 24, -0.02, 41, depth, 0.3))
    net.steps = 120
    state = {"written": False, "host": None}

    def check(model, oracle):
        compare_state(net, model, oracle, f"after {model.timestep} steps", exact=True)
        if not state["written"]:
            g = model.synapse_populations["AA"].vars["g"]
            lib = _abi.load()
            host = np.zeros(g.count, np.float32)                       # the caller's host buffer (never copied from here)
            state["host"] = host
            _abi.check(lib.gennmi_register_mirror(host.ctypes.data_as(C.c_void_p), C.c_void_p(g.ptr), host.nbytes))
            _abi.check(lib.gennmi_flush())
            staging = C.c_void_p()
            _abi.check(lib.gennmi_malloc(C.byref(staging), host.nbytes))
            new = np.full(g.count, -0.03, np.float32)
            _abi.check(lib.gennmi_memcpy_to_device(staging, new.ctypes.data_as(C.c_void_p), new.nbytes))
            hip = C.CDLL("libamdhip64.so")
            assert hip.hipMemcpy(C.c_void_p(g.ptr), staging, C.c_size_t(new.nbytes), C.c_int(3)) == 0      # hipMemcpyDeviceToDevice
            _abi.check(lib.gennmi_note_mirror_write(C.c_void_p(host.ctypes.data + 4 * 100)))               # a pointer INTO the host buffer
            lib.gennmi_free(staging)
            assert lib.gennmi_note_mirror_write(C.c_void_p(new.ctypes.data)) != 0                           # not a registered buffer
            _abi.check(lib.gennmi_unregister_mirror(host.ctypes.data_as(C.c_void_p)))
            oracle.syn_g("AA")[:] = np.float32(-0.03)
            state["written"] = True

    model, oracle, spikes = _run_chunks(net, (60, 60), check)
    assert model.runner_info()["resident_plan"]
    assert spikes > 500
    model.unload()


@pytest.mark.parametrize("limit, rows", [(64, 230), (1000, 230), (7, 230), (64, 50), (64, 0)])
def test_queued_single_steps_take_the_resident_launch(limit, rows):
    """step_time() one call at a time with the step queue on (what the reference's Runtime::stepTime amounts to): the steps
    run as resident launches of up to `limit` steps, cut wherever something looks at the device -- state pulls, a push
    of membrane potentials, the event counter, a recording buffer of `rows` rows that wraps -- and everything is as unqueued stepping leaves it."""
    n_a, n_b, depth = 700, 300, 7
    net = Net(name="resident_queue", dt=1.0, steps=230)
    net.pops.append(_pop("A", n_a, 0.62, -60.0 + 9.5 * rng.uniform(5, 1, 0, n_a)))
    net.pops.append(_pop("B", n_b, 0.45, -60.0 + 9.5 * rng.uniform(5, 2, 0, n_b)))
    net.syns.append(_projection("AB", "A", "B", n_a, n_b, 40, 0.11, 11, depth, 0.3))
    net.syns.append(_projection("BA", "B", "A", n_b, n_a, 64, -0.07, 12, depth, 0.3))
    model = model_from_net(net, record=bool(rows))
    model.load(num_recording_timesteps=rows or None)
    assert model.runner_info()["resident_plan"]
    model.set_step_queue(limit)
    oracle = OracleNet(net, num_recording_timesteps=rows)
    done = 0
    for chunk in (1, 2, 3, 40, 9, 100, 75):
        for _ in range(chunk):
            model.step_time()
        oracle.run(chunk)
        done += chunk
        if done == 55:
            # a push lands between the steps it was issued between (the steps queued before it have run by then)
            v = model.neuron_populations["B"].vars["V"]
            v.pull_from_device()
            v.view[::3] = np.float32(-50.5)
            v.push_to_device()
            oracle.var("B", 0)[::3] = np.float32(-50.5)
        elif done == 155:
            assert model.synaptic_event_count == oracle.events()
        else:
            compare_state(net, model, oracle, f"after {done} queued steps", exact=True)      # pulls, no synchronize() first
    assert done == net.steps
    if rows:
        model.pull_recording_buffers_from_device()
        for p in net.pops:
            assert np.array_equal(model.neuron_populations[p.name].vars["recordSpk"].view, oracle.record(p.name, rows)), f"recording of {p.name} differs"
    assert model.synaptic_event_count == oracle.events() and oracle.events() > 50000
    model.set_step_queue(0)
    model.unload()


def test_plan_can_be_switched_off(monkeypatch):
    monkeypatch.setenv("GENNMI_RESIDENT", "0")
    n, depth = 600, 4
    net = Net(name="resident_off", dt=1.0, steps=0)
    net.pops.append(_pop("A", n, 0.6, -60.0 + 9.5 * rng.uniform(7, 1, 0, n)))
    net.syns.append(_projection("AA", "A", "A", n, n, 48, 0.04, 31, depth, 0.4))
    net.steps = 120

    def check(model, oracle):
        compare_state(net, model, oracle, f"after {model.timestep} steps", exact=True)

    model, oracle, spikes = _run_chunks(net, (120,), check, resident=False)
    model.unload()


@pytest.mark.parametrize("resident", ["1", "0"])
def test_expired_wait_is_reported_not_hung(resident, monkeypatch):
    """Failure path, forced from the host: with a wait bound of zero polls the first word (resident plan) or spike
    count (per-step plans) that has not arrived when it is first looked at makes the work-group raise the device error
    flag and leave; every kernel still ends normally, and the next synchronisation reports the error."""
    from genn_amd import configs
    from genn_amd._abi import GennmiError
    monkeypatch.setenv("GENNMI_SPIN_LIMIT", "0")
    monkeypatch.setenv("GENNMI_RESIDENT", resident)
    net = configs.potjans(neuron_scale=0.05, connectivity_scale=1.0, steps=2000)
    model = model_from_net(net)
    model.load(num_recording_timesteps=2000)
    assert model.runner_info()["resident_plan"] == (resident == "1")
    model.run(2000)
    with pytest.raises(GennmiError, match="bounded wait"):
        model.synchronize()
    model.unload()
    # the bound is per process: restore the default for whatever runs next
    monkeypatch.delenv("GENNMI_SPIN_LIMIT")
    model = model_from_net(net)
    model.load(num_recording_timesteps=100)
    model.run(100)
    model.synchronize()
    model.unload()
