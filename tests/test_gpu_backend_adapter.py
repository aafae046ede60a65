"""The GeNN backend adapter end to end, on the GPU: the reference's OWN model description, code generator and
Runtime (libgenn, compiled from the reference tree into oracle/_ref/) drive the MI355X device library through
`GeNN::CodeGenerator::MI355X::Backend` (genn_amd/backend/).  oracle/_ref/mi355x_driver builds each golden case as a
ModelSpec, selects the MI355X backend, generates and compiles the runner, and steps it with Runtime::stepTime;
its dumps are compared with the fixtures that the reference's SingleThreadedCPU backend produced for the same
inputs (tests/golden/*.npz): spike rasters identical, state within 1e-5 (bit-exact where no sum can be reordered),
column remap bit-exact.

Needs the prebuilt driver (built where the reference tree is mounted) and g++/make for the generated runner.
"""
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

from cases import CASES, REFERENCE_ONLY  # noqa: E402
from genn_amd.netspec import write_netspec  # noqa: E402

DRIVER = os.path.join(ROOT, "oracle", "_ref", "mi355x_driver")
pytestmark = [pytest.mark.gpu,
              pytest.mark.skipif(not os.path.exists(DRIVER), reason="oracle/_ref/mi355x_driver is not built (needs the reference tree at build time)")]

REL_TOL = 1e-5


def _close(got, want, what, accumulator=False):
    floor = max(1e-3, float(np.abs(want).max(initial=0.0))) if accumulator else 1e-3
    err = np.abs(got.astype(np.float64) - want.astype(np.float64)) / np.maximum(np.abs(want), floor)
    assert err.max(initial=0.0) <= REL_TOL, f"{what}: max relative error {err.max():.3e}"


def _run(case, *options):
    net, snap = CASES[case]()
    net.snap = snap
    tmp = tempfile.mkdtemp(prefix="adapter_")
    spec, work, out = (os.path.join(tmp, d) for d in ("spec", "work", "out"))
    for d in (work, out):
        os.makedirs(d)
    write_netspec(net, spec)
    print(f"adapter case {case}: running {DRIVER}", flush=True)
    res = subprocess.run([DRIVER, spec, work, out, *options], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=240,
                         env=dict(os.environ, GENNMI_PROGRAM_STATS="1"))
    assert res.returncode == 0, res.stdout[-3000:]
    code = os.path.join(work, net.name + "_CODE")
    net.generated_kernels = "__global__" in open(os.path.join(code, "neuronUpdate.cc")).read()
    net.driver_output = res.stdout
    return net, snap, tmp, out


def _program_stats(output):
    """calls of updateSynapses / updateNeurons executed by the runner's program, how many of them replayed from a captured
    graph, launches made, graphs captured (printed by the device library when the program is destroyed)"""
    import re
    m = re.search(r"gennmi_program: calls (\d+), replayed (\d+), launches (\d+), graphs (\d+)", output)
    assert m, output[-2000:]
    return tuple(int(g) for g in m.groups())


# cases whose models the device library implements; the others (models of the test driver's own, parameters set while the
# model runs) take generated kernels by themselves
LIBRARY_CASES = sorted(set(CASES) - REFERENCE_ONLY)
# what the generated kernels cover: SPARSE / DENSE matrices, any neuron, postsynaptic, current-source and weight-update code
# without delay slots, spike-like events or random numbers
GENERATED_CASES = ["va_double_small", "post_events_small", "custom_small", "dynamic_small", "synapse_dynamics_small", "prev_times_small", "stdp_delay_small", "va_delay_small", "graded_small", "conv_small", "dense_small", "va_small", "potjans_small", "izhikevich_small", "stdp_small", "stdp_additive_small", "reverse_small"]


@pytest.mark.parametrize("case", LIBRARY_CASES)
def test_adapter_matches_reference_backend(case):
    _compare_with_fixture(case)


@pytest.mark.parametrize("case", GENERATED_CASES)
def test_generated_kernels_match_reference_backend(case):
    """Kernels GENERATED from the model's own code strings (Preferences::kernelSource): GeNN's environments print the
    snippets into this backend's skeletons, hipcc compiles the module for gfx950 as part of the runner, and the reference's
    Runtime steps it.  `custom_small` is a network of models that exist nowhere but in the test driver — LIF neurons with
    an extra state variable, a weight-update model with presynaptic and postsynaptic variables after
    tests/features/test_wu_vars.py — and takes this path by itself; so does `dynamic_small`, whose parameters change
    while it runs (Runtime::setDynamicParamValue, after tests/features/test_dynamic_param.py).  The other cases are forced onto it, so every fixture the
    reference's CPU backend produced for a covered feature (dendritic delay, trace and built-in STDP with learnPost,
    presynaptic output, an array-fed current source) also pins the generated kernels."""
    _compare_with_fixture(case, "--kernels=generated")


@pytest.mark.parametrize("case", ["potjans_small", "stdp_small", "custom_small", "stdp_delay_small", "dynamic_small"])
@pytest.mark.parametrize("queue", [8, 0])
def test_generated_kernels_replayed_from_a_graph_match_reference_backend(case, queue):
    """Runtime::stepTime asks for one step at a time; the runner's program notes the calls of updateSynapses / updateNeurons
    and replays a full queue from a captured graph whose kernels read their step's time, recording row, random-number step and
    look-back tag from a device table.  With a queue of 8 steps most of a run is replayed (what is left when the driver takes
    a snapshot is launched call by call); with no queue every call is launched when made.  Either way the fixtures of the
    reference's CPU backend must be met exactly as with the default queue, replay after replay."""
    net = _compare_with_fixture(case, "--kernels=generated", f"--step-queue={queue}")
    calls, replayed, launches, graphs = _program_stats(net.driver_output)
    assert calls == 2 * net.steps, (calls, net.steps)
    if queue:
        assert graphs >= 1 and replayed >= calls // 2 and replayed % (2 * queue) == 0, (calls, replayed, graphs)
    else:
        assert graphs == 0 and replayed == 0


def test_generated_kernels_report_an_expired_wait():
    """Failure path of the generated spike compaction, forced from the host (a wait bound of zero polls): the work-group that
    finds another one's count not yet published raises the program's error flag and leaves, every kernel ends normally, and
    the next call that waits for the device — here the driver's first pull — reports it, whatever the model's timing setting
    (timing is off here).  The run must fail with that message instead of going on with undefined spike queues."""
    from genn_amd import configs
    net = configs.potjans(neuron_scale=0.05, connectivity_scale=0.2, steps=200)
    net.snap = 100
    tmp = tempfile.mkdtemp(prefix="adapter_expired_")
    try:
        spec, work, out = (os.path.join(tmp, d) for d in ("spec", "work", "out"))
        for d in (work, out):
            os.makedirs(d)
        write_netspec(net, spec)
        print("adapter: generated kernels with a wait bound of zero", flush=True)
        res = subprocess.run([DRIVER, spec, work, out, "--kernels=generated"], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=240,
                             env=dict(os.environ, GENNMI_SPIN_LIMIT="0"))
        assert res.returncode != 0 and "bounded wait" in res.stdout, res.stdout[-3000:]
        print("adapter: the same run with the default bound", flush=True)
        res = subprocess.run([DRIVER, spec, work, out, "--kernels=generated"], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=240)
        assert res.returncode == 0, res.stdout[-3000:]
    finally:
        shutil.rmtree(tmp, ignore_errors=True)


def _compare_with_fixture(case, *options):
    golden = np.load(os.path.join(HERE, "golden", case + ".npz"))
    net, snap, tmp, out = _run(case, *options)
    try:
        # (custom_update_*: built-in snippets, so the step keeps the library's kernels; only its custom updates are generated)
        assert net.generated_kernels == ("--kernels=generated" in options or (case in REFERENCE_ONLY and not case.startswith("custom_update_")))
        assert str(golden["input_digest"]) == net.input_digest(), "generator output changed since the fixture was made"
        exact = (case == "va_small")
        spikes = 0
        for p in net.pops:
            got = np.fromfile(os.path.join(out, f"{p.name}.spikes.u32"), np.uint32).reshape(-1, 2)
            want = golden[f"spikes.{p.name}"]
            assert np.array_equal(got, want), f"raster of {p.name} differs ({len(got)} vs {len(want)} spikes)"
            spikes += len(want)
            for var in ("V", "RefracTime", "U", "A"):
                key = f"{var}.{p.name}"
                if key in golden:
                    g = np.fromfile(os.path.join(out, f"{p.name}.{var}.f32"), np.float32).reshape(-1, p.n)
                    if exact:
                        assert np.array_equal(g, golden[key]), f"{key} differs"
                    elif net.precision == "double":
                        # fp64 on both sides, dumped as fp32: a rounding step apart at most (computed in fp32 the same values are
                        # 4e-6 off, which the general tolerance would let through)
                        err = np.abs(g.astype(np.float64) - golden[key]) / np.maximum(np.abs(golden[key]), 1e-3)
                        assert err.max() <= 2.5e-7, f"{key}: max relative error {err.max():.3e}"
                    else:
                        _close(g, golden[key], key)
        assert spikes > 50
        # recorded spike-like events, where the fixture holds them
        for s in net.syns:
            if f"events.{s.name}" in golden:
                got = np.fromfile(os.path.join(out, f"{s.name}.events.u32"), np.uint32).reshape(-1, 2)
                assert np.array_equal(got, golden[f"events.{s.name}"]), f"recorded events of {s.name} differ"

        # (projections rewired while the model ran: their final weights are compared within the final rows, their column view
        # is the one dumped before the first step)
        rewired_final = {c.target: (np.arange(net.syn(c.target).row_stride)[None, :] < golden[f"custom.{c.name}.rowLength"][-1][:, None]).reshape(-1)
                         for c in net.customs if f"custom.{c.name}.rowLength" in golden.files}
        for s in net.syns:
            for var in ("colLength", "remap"):
                key = f"{var}.{s.name}"
                if key in golden:
                    got = np.fromfile(os.path.join(out, f"{s.name}.{var}.u32"), np.uint32)
                    if var == "colLength":
                        assert np.array_equal(got, golden[key]), key
                    else:
                        stride = int(golden[f"colStride.{s.name}"])
                        length = golden[f"colLength.{s.name}"]
                        mask = np.arange(stride)[None, :] < length[:, None]
                        assert np.array_equal(got.reshape(-1, stride)[mask], golden[key].reshape(-1, stride)[mask]), key
            for var in ("sPre", "sPost", "wPre", "wPost"):
                # spike times copied around by the weight-update code of custom_small: exact values, nothing is summed
                key = f"{var}.{s.name}"
                if key in golden:
                    got = np.fromfile(os.path.join(out, f"{s.name}.{var}.f32"), np.float32).reshape(net.steps // snap, -1)
                    assert np.array_equal(got, golden[key]), key
            if f"hits.{s.name}" in golden:
                # steps counted per synapse by postsynaptic spike-like events (within the rows: their padding is never initialised)
                valid = (np.arange(s.row_stride)[None, :] < s.row_length[:, None]).reshape(-1)
                got = np.fromfile(os.path.join(out, f"{s.name}.hits.f32"), np.float32).reshape(net.steps // snap, -1)
                assert np.array_equal(got[:, valid], golden[f"hits.{s.name}"][:, valid]), f"hits.{s.name}"
                assert got[-1, valid].sum() > 1000
            for var in ("g", "preTrace", "postTrace", "outPost", "x"):
                key = f"{var}.{s.name}"
                if key in golden:
                    got = np.fromfile(os.path.join(out, f"{s.name}.{var}.f32"), np.float32).reshape(net.steps // snap, -1)
                    want = golden[key]
                    got = got[-1] if want.ndim == 1 else got
                    if var == "g" and s.name in rewired_final:
                        got, want = got[rewired_final[s.name]], want[rewired_final[s.name]]
                    _close(got, want, key, accumulator=(var == "outPost"))
        # variables of custom updates and what the updates wrote into the arrays they refer to, snapshot by snapshot
        # (a projection that custom connectivity updates rewire: row lengths exact, everything on its synapses within the rows)
        rewired = {c.target: golden[f"custom.{c.name}.rowLength"] for c in net.customs if f"custom.{c.name}.rowLength" in golden.files}
        masks = {target: (np.arange(net.syn(target).row_stride)[None, None, :] < lengths[:, :, None]).reshape(len(lengths), -1) for target, lengths in rewired.items()}
        for key in golden.files:
            if key.startswith("custom."):
                _, name, var = key.split(".")
                target = next(c.target for c in net.customs if c.name == name)
                want = golden[key]
                if want.dtype == np.uint32:
                    got = np.fromfile(os.path.join(out, f"{name}.{var}.u32"), np.uint32).reshape(net.steps // snap, -1)
                    if var == "ind":
                        assert np.array_equal(got[masks[target]], want[masks[target]]), key
                    else:
                        assert np.array_equal(got, want), key
                    continue
                got = np.fromfile(os.path.join(out, f"{name}.{var}.f32"), np.float32).reshape(net.steps // snap, -1)
                if target in masks and got.shape == masks[target].shape:
                    got, want = got[masks[target]], want[masks[target]]
                if var in ("applied", "when", "removed", "born"):
                    # call counts, the time handed to the update, when a synapse was made: nothing is summed
                    assert np.array_equal(got, want), key
                _close(got, want, key)
        for s in net.syns:
            key = f"denDelay.{s.name}"
            if key in golden:
                D, n = s.max_den_delay, net.pop(s.trg).n
                got = np.fromfile(os.path.join(out, f"{s.name}.denDelay.f32"), np.float32).reshape(net.steps // snap, -1)[-1].reshape(D, n).copy()
                want = golden[key].reshape(D, n).copy()
                if not net.generated_kernels:
                    # single-launch step: the slot read next already holds the zero-delay input of the last step's spikes
                    nxt = (net.steps + 1) % D
                    got[nxt] = 0
                    want[nxt] = 0
                _close(got, want, key, accumulator=True)
    finally:
        shutil.rmtree(tmp, ignore_errors=True)
    return net


def test_adapter_full_size_microcircuit_first_100ms():
    """77,169 neurons / 298,624,465 synapses through the reference's Runtime::stepTime on the MI355X backend, 1000
    steps: rasters must be those of the CPU oracle, final membrane potentials within 1e-5."""
    from genn_amd import configs
    from oracle.genn_cpu import OracleNet
    net = configs.potjans(steps=1000)
    net.snap = 0
    tmp = tempfile.mkdtemp(prefix="adapter_full_")
    try:
        spec, work, out = (os.path.join(tmp, d) for d in ("spec", "work", "out"))
        for d in (work, out):
            os.makedirs(d)
        write_netspec(net, spec)
        print(f"adapter full-size microcircuit: running {DRIVER}", flush=True)
        res = subprocess.run([DRIVER, spec, work, out], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=280)
        assert res.returncode == 0, res.stdout[-3000:]
        oracle = OracleNet(net, num_recording_timesteps=net.steps)
        oracle.run(net.steps)
        total = 0
        for p in net.pops:
            got = np.fromfile(os.path.join(out, f"{p.name}.spikes.u32"), np.uint32).reshape(-1, 2)
            words = (p.n + 31) // 32
            bits = np.unpackbits(oracle.record(p.name, net.steps).view(np.uint8).reshape(net.steps, words * 4), axis=1, bitorder="little")[:, :p.n]
            steps, ids = np.nonzero(bits)
            want = np.stack([steps, ids], axis=1).astype(np.uint32)
            assert np.array_equal(got, want), f"raster of {p.name} differs ({len(got)} vs {len(want)} spikes)"
            total += len(want)
            v = np.fromfile(os.path.join(out, f"{p.name}.V.f32"), np.float32)
            _close(v, oracle.var(p.name, 0), f"V of {p.name}")
        assert total > 10000
        oracle.close()
    finally:
        shutil.rmtree(tmp, ignore_errors=True)


def test_adapter_batched_toeplitz_layer():
    """Batch size 3 through the adapter (the reference's CPU backend has no batch): shared kernel weights and spike
    times, per-batch spike-source windows; batch b must equal a batch-1 oracle run fed batch b's input."""
    import copy
    from genn_amd import configs
    from oracle.genn_cpu import OracleNet
    B = 3
    nets = [configs.conv_toeplitz(h=8, w=8, ic=2, oc=4, steps=60, w_sd=0.6, batch_index=b, ioffset=0.4) for b in range(B)]
    times = np.concatenate([n.pop("In").spike_times for n in nets])
    offs = np.cumsum([0] + [len(n.pop("In").spike_times) for n in nets])
    batched = copy.deepcopy(nets[0])
    batched.pop("In").vars = {"startSpike": np.stack([n.pop("In").vars["startSpike"] + offs[b] for b, n in enumerate(nets)]).astype(np.uint32),
                              "endSpike": np.stack([n.pop("In").vars["endSpike"] + offs[b] for b, n in enumerate(nets)]).astype(np.uint32)}
    batched.pop("In").spike_times = times
    batched.batch_size = B
    batched.snap = 0
    tmp = tempfile.mkdtemp(prefix="adapter_batch_")
    try:
        spec, work, out = (os.path.join(tmp, d) for d in ("spec", "work", "out"))
        for d in (work, out):
            os.makedirs(d)
        write_netspec(batched, spec)
        print(f"adapter batched conv: running {DRIVER}", flush=True)
        res = subprocess.run([DRIVER, spec, work, out], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=240)
        assert res.returncode == 0, res.stdout[-3000:]
        total = 0
        for b, net in enumerate(nets):
            oracle = OracleNet(net, num_recording_timesteps=net.steps)
            oracle.run(net.steps)
            for p in net.pops:
                got = np.fromfile(os.path.join(out, f"{p.name}.spikes{'.b%d' % b if b else ''}.u32"), np.uint32).reshape(-1, 2)
                words = (p.n + 31) // 32
                bits = np.unpackbits(oracle.record(p.name, net.steps).view(np.uint8).reshape(net.steps, words * 4), axis=1, bitorder="little")[:, :p.n]
                steps, ids = np.nonzero(bits)
                assert np.array_equal(got, np.stack([steps, ids], axis=1).astype(np.uint32)), f"batch {b}: raster of {p.name} differs"
                total += len(ids)
            n_out = net.pop("Out").n
            v = np.fromfile(os.path.join(out, "Out.V.f32"), np.float32).reshape(-1, B, n_out)[-1, b]
            _close(v, oracle.var("Out", 0), f"batch {b}: V of Out")
            oracle.close()
        assert total > 300
    finally:
        shutil.rmtree(tmp, ignore_errors=True)


def test_adapter_batched_plastic_network():
    """Batch size 2 with trace STDP through the adapter: the Runtime duplicates the weights (VarAccess::READ_WRITE), the traces
    and the spike times per batch; the batches differ in initial membrane potentials and Poisson spike trains, and batch b
    must equal a batch-1 oracle run on batch b's inputs, final weights included."""
    import copy
    from genn_amd import configs, rng
    from genn_amd.configs import poisson_spike_source
    from oracle.genn_cpu import OracleNet
    B, steps = 2, 100
    nets = []
    for b in range(B):
        net = configs.plastic_stdp(n=1500, n_src=100, steps=steps, fan=80, src_fan=60)
        if b:
            for k, name in enumerate(("E", "I")):
                p = net.pop(name)
                p.vars["V"] = (-60.0 + 10.0 * rng.uniform(4321 + b, 1 + k, 0, p.n)).astype(np.float32)
            start, end, times = poisson_spike_source(net.seed, 70 + b, 100, 10.0, steps, net.dt)
            net.pop("P").vars = {"startSpike": start, "endSpike": end}
            net.pop("P").spike_times = times
        nets.append(net)
    batched = copy.deepcopy(nets[0])
    for name in ("E", "I"):
        batched.pop(name).vars = {"V": np.stack([n.pop(name).vars["V"] for n in nets]), "RefracTime": np.zeros((B, nets[0].pop(name).n), np.float32)}
    offs = np.cumsum([0] + [len(n.pop("P").spike_times) for n in nets])
    batched.pop("P").vars = {"startSpike": np.stack([n.pop("P").vars["startSpike"] + offs[b] for b, n in enumerate(nets)]).astype(np.uint32),
                             "endSpike": np.stack([n.pop("P").vars["endSpike"] + offs[b] for b, n in enumerate(nets)]).astype(np.uint32)}
    batched.pop("P").spike_times = np.concatenate([n.pop("P").spike_times for n in nets])
    batched.batch_size = B
    batched.snap = 0
    tmp = tempfile.mkdtemp(prefix="adapter_batch_stdp_")
    try:
        spec, work, out = (os.path.join(tmp, d) for d in ("spec", "work", "out"))
        for d in (work, out):
            os.makedirs(d)
        write_netspec(batched, spec)
        print(f"adapter batched plastic network: running {DRIVER}", flush=True)
        res = subprocess.run([DRIVER, spec, work, out], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=240)
        assert res.returncode == 0, res.stdout[-3000:]
        total = 0
        g = np.fromfile(os.path.join(out, "EE.g.f32"), np.float32).reshape(B, -1)
        for b, net in enumerate(nets):
            oracle = OracleNet(net, num_recording_timesteps=net.steps)
            oracle.run(net.steps)
            for p in net.pops:
                got = np.fromfile(os.path.join(out, f"{p.name}.spikes{'.b%d' % b if b else ''}.u32"), np.uint32).reshape(-1, 2)
                words = (p.n + 31) // 32
                bits = np.unpackbits(oracle.record(p.name, net.steps).view(np.uint8).reshape(net.steps, words * 4), axis=1, bitorder="little")[:, :p.n]
                steps_, ids = np.nonzero(bits)
                assert np.array_equal(got, np.stack([steps_, ids], axis=1).astype(np.uint32)), f"batch {b}: raster of {p.name} differs"
                total += len(ids)
            assert np.array_equal(g[b], oracle.syn_g("EE").reshape(-1)), f"batch {b}: weights differ"
            oracle.close()
        assert total > 1000 and not np.array_equal(g[0], g[1])
    finally:
        shutil.rmtree(tmp, ignore_errors=True)


def test_generated_kernels_with_batches():
    """Batch size 2 for models only the generated kernels cover (`custom_small`: a neuron with an extra state variable, a
    weight-update model with presynaptic, postsynaptic and per-synapse variables): the batch is the grid's second
    dimension, every batch compacts its own spike queue, and GeNN's own index helpers place variables by their batch
    dimension.  The reference's CPU backend has no batches, so batch b is pinned by that backend's run from batch b's
    initial values (fixtures `custom_small` and `custom_batch1_small`): rasters identical, spike times copied through the
    weight-update variables exact, state within 1e-5."""
    import copy
    B = 2
    cases = ("custom_small", "custom_batch1_small")
    nets, snap = [], None
    for case in cases:
        net, snap = CASES[case]()
        nets.append(net)
    batched = copy.deepcopy(nets[0])
    for p in batched.pops:
        p.vars = {v: np.stack([n.pop(p.name).vars[v] for n in nets]) for v in p.vars}
    batched.batch_size = B
    batched.snap = snap
    tmp = tempfile.mkdtemp(prefix="adapter_batch_generated_")
    try:
        spec, work, out = (os.path.join(tmp, d) for d in ("spec", "work", "out"))
        for d in (work, out):
            os.makedirs(d)
        write_netspec(batched, spec)
        print(f"adapter batched generated kernels: running {DRIVER}", flush=True)
        res = subprocess.run([DRIVER, spec, work, out], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=240)
        assert res.returncode == 0, res.stdout[-3000:]
        assert "__global__" in open(os.path.join(work, batched.name + "_CODE", "neuronUpdate.cc")).read()
        snaps = batched.steps // snap
        for b, case in enumerate(cases):
            golden = np.load(os.path.join(HERE, "golden", case + ".npz"))
            assert str(golden["input_digest"]) == nets[b].input_digest(), "generator output changed since the fixture was made"
            spikes = 0
            for p in batched.pops:
                got = np.fromfile(os.path.join(out, f"{p.name}.spikes{'.b%d' % b if b else ''}.u32"), np.uint32).reshape(-1, 2)
                want = golden[f"spikes.{p.name}"]
                assert np.array_equal(got, want), f"batch {b}: raster of {p.name} differs ({len(got)} vs {len(want)} spikes)"
                spikes += len(want)
                for var in ("V", "RefracTime", "A"):
                    g = np.fromfile(os.path.join(out, f"{p.name}.{var}.f32"), np.float32).reshape(snaps, B, p.n)[:, b]
                    _close(g, golden[f"{var}.{p.name}"], f"batch {b}: {var}.{p.name}")
            assert spikes > 500
            for s in batched.syns:
                for var in ("sPre", "sPost", "wPre", "wPost"):
                    key = f"{var}.{s.name}"
                    if key in golden:
                        got = np.fromfile(os.path.join(out, f"{s.name}.{var}.f32"), np.float32).reshape(snaps, B, -1)[:, b]
                        assert np.array_equal(got, golden[key]), f"batch {b}: {key}"
                got = np.fromfile(os.path.join(out, f"{s.name}.outPost.f32"), np.float32).reshape(snaps, B, -1)[:, b]
                _close(got, golden[f"outPost.{s.name}"], f"batch {b}: outPost.{s.name}", accumulator=True)
    finally:
        shutil.rmtree(tmp, ignore_errors=True)


def test_custom_updates_match_reference_backend():
    """Custom updates (Runtime::customUpdate, after tests/features/test_custom_update.py): update groups called every 20, 30
    and 50 steps while the network runs — a per-neuron update of the membrane potentials with a variable of its own, sum and
    maximum over a population, weight decay over a plastic SPARSE and a static DENSE matrix with per-synapse variables,
    the decayed dense matrix transposed into another projection's weights, and a reduction over batches.  The custom
    updates' kernels are generated from their code; the step runs on the device library's kernels (the model's snippets are
    built-in ones), which are told what the updates wrote.  Rasters identical to the reference CPU backend's, call counts
    and the time handed to the update code exact, everything else within 1e-5."""
    _compare_with_fixture("custom_update_small")


@pytest.mark.parametrize("options", [(), ("--step-queue=0",), ("--kernels=generated",)], ids=["queued_steps", "step_by_step", "generated_step"])
def test_custom_updates_between_queued_resident_steps(options):
    """Custom updates over a static network without delays, which the device library steps on its resident plan with
    Runtime::stepTime calls queued: every 40 steps the weights of a static projection decay (the library keeps packed
    copies of them), every 25 one population's potentials are pulled towards rest (the resident kernel keeps them in
    registers while it runs).  The queued steps must have run before an update launches and the copies must be rebuilt
    after it: rasters identical to the reference CPU backend's, with the queue, with every step launched when asked
    for, and on generated kernels."""
    _compare_with_fixture("custom_update_static_small", *options)


def test_custom_connectivity_updates_match_reference_backend():
    """Structural plasticity (custom connectivity updates, after tests/features/test_custom_connectivity_update.py) in a
    learning network: every 40 steps synapses whose weight has fallen below a threshold are removed — the row's last synapse
    moves into the gap together with the learned weight and the per-synapse variables of two other custom updates — and every
    25 steps each row with room sprouts a synapse; the projection learns from postsynaptic spikes, so its column view is
    rebuilt after every change.  Such a model takes generated kernels by itself (the device library's launch plans rely on
    rows sorted by target).  Row lengths, targets, removal counts and birth times identical to the reference CPU backend's at
    every snapshot, rasters identical, weights and accumulators within 1e-5."""
    _compare_with_fixture("rewiring_small")


def test_custom_updates_match_reference_backend_on_generated_kernels():
    """The same with the step's kernels generated too (what a model of the user's own snippets gets)."""
    _compare_with_fixture("custom_update_small", "--kernels=generated")


@pytest.mark.parametrize("options", [(), ("--kernels=generated",)], ids=["library_step", "generated_step"])
def test_custom_updates_with_batches(options):
    """The same network with batch size 3, the step on the library's kernels or on generated ones.  The reference's CPU backend has no batches, so batch 0 (same initial values) is
    pinned by its fixture, and what batches add by closed forms: the reduction over neurons gives every batch the sum and
    maximum of ITS membrane potentials, the reduction over batches the sum and maximum of the per-batch plastic weights,
    the static dense weights (shared between batches) decay once per call, not once per batch."""
    import copy
    B = 3
    net, snap = CASES["custom_update_small"]()
    golden = np.load(os.path.join(HERE, "golden", "custom_update_small.npz"))
    assert str(golden["input_digest"]) == net.input_digest(), "generator output changed since the fixture was made"
    batched = copy.deepcopy(net)
    from genn_amd import rng
    for k, p in enumerate(batched.pops):
        other = [(-60.0 + 9.5 * rng.uniform(net.seed, 71 + 2 * k + b, 0, p.n)).astype(np.float32) for b in range(B - 1)]
        p.vars = {"V": np.stack([p.vars["V"]] + other), "RefracTime": np.zeros((B, p.n), np.float32)}
    batched.batch_size = B
    batched.snap = snap
    tmp = tempfile.mkdtemp(prefix="adapter_custom_batched_")
    try:
        spec, work, out = (os.path.join(tmp, d) for d in ("spec", "work", "out"))
        for d in (work, out):
            os.makedirs(d)
        write_netspec(batched, spec)
        print(f"adapter batched custom updates: running {DRIVER} {' '.join(options)}", flush=True)
        res = subprocess.run([DRIVER, spec, work, out, *options], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=240)
        assert res.returncode == 0, res.stdout[-3000:]
        snaps = batched.steps // snap
        load = lambda name: np.fromfile(os.path.join(out, name), np.float32)        # noqa: E731
        # batch 0 against the fixture
        for p in batched.pops:
            got = np.fromfile(os.path.join(out, f"{p.name}.spikes.u32"), np.uint32).reshape(-1, 2)
            assert np.array_equal(got, golden[f"spikes.{p.name}"]), f"batch 0: raster of {p.name} differs"
            other = np.fromfile(os.path.join(out, f"{p.name}.spikes.b1.u32"), np.uint32).reshape(-1, 2)
            assert len(other) > 100 and not np.array_equal(other, got)
            _close(load(f"{p.name}.V.f32").reshape(snaps, B, p.n)[:, 0], golden[f"V.{p.name}"], f"batch 0: V.{p.name}")
        assert np.array_equal(load("BDecay.applied.f32").reshape(snaps, B, -1)[:, 0], golden["custom.BDecay.applied"])
        assert np.array_equal(load("BDecay.applied.f32").reshape(snaps, B, -1)[:, 2], golden["custom.BDecay.applied"])
        _close(load("PlasticDecay.w.f32").reshape(snaps, B, -1)[:, 0], golden["custom.PlasticDecay.w"], "batch 0: plastic weights")
        _close(load("PlasticDecay.total.f32").reshape(snaps, B, -1)[:, 0], golden["custom.PlasticDecay.total"], "batch 0: PlasticDecay.total")
        # shared between batches: one copy, decayed once per call
        for var in ("w", "total", "when"):
            _close(load(f"DenseDecay.{var}.f32").reshape(snaps, -1), golden[f"custom.DenseDecay.{var}"], f"DenseDecay.{var}")
        _close(load("Feedback.transposed.f32").reshape(snaps, -1), golden["custom.Feedback.transposed"], "Feedback.transposed")
        # reduction over neurons, per batch: the calls after steps 100 and 200 coincide with snapshots, and nothing writes A's V
        # between the call and the snapshot
        V = load("A.V.f32").reshape(snaps, B, -1).astype(np.float64)
        total, peak = load("ASum.sum.f32").reshape(snaps, B), load("ASum.peak.f32").reshape(snaps, B)
        for k in (1, 3):
            assert np.allclose(total[k], V[k].sum(axis=1), rtol=2e-6) and np.array_equal(peak[k], V[k].max(axis=1).astype(np.float32))
        assert len(set(total[3].tolist())) == B
        # reduction over batches: every snapshot follows a call (both every 50 steps)
        w = load("PlasticReduce.w.f32").reshape(snaps, B, -1)
        mask = (np.arange(net.syn("AB_plastic").row_stride)[None, :] < net.syn("AB_plastic").row_length[:, None]).reshape(-1)
        assert np.abs(w[-1, 0] - w[-1, 1])[mask].max() > 1e-3           # the batches' weights have diverged
        got_sum, got_peak = load("PlasticReduce.sum.f32").reshape(snaps, -1), load("PlasticReduce.peak.f32").reshape(snaps, -1)
        assert np.allclose(got_sum[:, mask], w.astype(np.float64).sum(axis=1)[:, mask], rtol=1e-6, atol=1e-7)
        assert np.array_equal(got_peak[:, mask], w.max(axis=1)[:, mask])
    finally:
        shutil.rmtree(tmp, ignore_errors=True)


def test_generated_kernels_on_procedural_matrices():
    """PROCEDURAL connectivity on generated kernels: a row is the connectivity snippet's own row build code, run afresh for
    every spike with random numbers from a counter-based generator keyed by (seed, projection, row, lane).  No backend of the
    reference draws the same numbers (its CPU backend has no procedural matrices at all), so this is **parity unpinned**
    against the reference and held to what the construction fixes instead.  Eight sources fire together twice, ten steps
    apart, through FixedProbability(0.1) with a dyadic weight into a DeltaCurr input of 1000 silent LIF neurons, four lanes
    per row: every target must receive exactly the same number of inputs both times (the matrix is a function of the seed,
    not of the step), the number of synapses must be Binomial(8000, 0.1), and no target outside a lane's share may be hit
    twice by one row.  Then the recurrent procedural network of the library tests (all four snippets, dyadic weights):
    identical rasters from two runs, population rates within 15 % of the device library's own procedural path."""
    from genn_amd import configs
    from genn_amd.netspec import Net, Pop, Syn
    n_src, n_trg, p_conn, g = 8, 1000, 0.1, 0.25
    lif = dict(C=1.0, TauM=20.0, Vrest=-60.0, Vreset=-60.0, Vthresh=1e9, Ioffset=0.0, TauRefrac=2.0)
    net = Net(name="procedural_rows", dt=1.0, steps=14, seed=4242)
    net.pops.append(Pop("S", "ssa", n_src, {}, {"startSpike": (2 * np.arange(n_src)).astype(np.uint32), "endSpike": (2 * np.arange(n_src) + 2).astype(np.uint32)},
                        spike_times=np.tile(np.array([1.0, 11.0], np.float32), n_src)))
    net.pops.append(Pop("T", "lif", n_trg, lif, {"V": np.full(n_trg, -60.0, np.float32), "RefracTime": np.zeros(n_trg, np.float32)}))
    net.syns.append(Syn("ST", "S", "T", matrix="procedural", wum="static_const", wum_params={"g": g}, psm="deltacurr",
                        connect=("FixedProbability", {"prob": p_conn}), threads_per_spike=4))
    net.snap = 1

    def run(network, *options):
        tmp = tempfile.mkdtemp(prefix="adapter_proc_generated_")
        spec, work, out = (os.path.join(tmp, d) for d in ("spec", "work", "out"))
        for d in (work, out):
            os.makedirs(d)
        write_netspec(network, spec)
        print(f"adapter procedural on generated kernels: running {DRIVER} {' '.join(options)}", flush=True)
        res = subprocess.run([DRIVER, spec, work, out, *options], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=240)
        assert res.returncode == 0, res.stdout[-3000:]
        generated = "__global__" in open(os.path.join(work, network.name + "_CODE", "neuronUpdate.cc")).read()
        return tmp, out, generated

    tmp, out, generated = run(net, "--kernels=generated")
    try:
        assert generated
        V = np.fromfile(os.path.join(out, "T.V.f32"), np.float32).reshape(net.steps, n_trg).astype(np.float64)
        rest, decay = -60.0, np.exp(-1.0 / 20.0)
        quantum = (1.0 - decay) * 20.0 * g                  # what one input adds to V (Rmembrane = TauM / C)
        moved = [k for k in range(net.steps) if np.any(V[k] != rest)]
        first = moved[0]
        hits1 = (V[first] - rest) / quantum
        hits2 = (V[first + 10] - rest - decay * (V[first + 9] - rest)) / quantum
        assert np.abs(hits1 - np.rint(hits1)).max() < 1e-3 and np.abs(hits2 - np.rint(hits2)).max() < 1e-3
        hits1, hits2 = np.rint(hits1).astype(int), np.rint(hits2).astype(int)
        assert np.array_equal(hits1, hits2), "the rows differ between the two times they were built"
        total = hits1.sum()
        sd = np.sqrt(n_src * n_trg * p_conn * (1 - p_conn))
        assert abs(total - n_src * n_trg * p_conn) < 4 * sd, f"{total} synapses in {n_src} rows of {n_trg} at p = {p_conn}"
        assert hits1.max() <= n_src and (hits1 > 0).sum() > 400
        # every lane's share of the target range got its part
        for lane in range(4):
            share = hits1[lane * 250:(lane + 1) * 250].sum()
            assert abs(share - total / 4) < 4 * sd / 2 + 1, f"lane {lane}: {share} of {total} synapses"
    finally:
        shutil.rmtree(tmp, ignore_errors=True)

    recurrent = configs.procedural(order_free=True)
    recurrent.steps, recurrent.snap = 100, 100
    counts = {}
    rasters = {}
    for label, options in (("generated", ("--kernels=generated",)), ("again", ("--kernels=generated",)), ("library", ())):
        tmp, out, generated = run(recurrent, *options)
        try:
            assert generated == (label != "library")
            rasters[label] = {p.name: np.fromfile(os.path.join(out, f"{p.name}.spikes.u32"), np.uint32).reshape(-1, 2) for p in recurrent.pops}
            counts[label] = {name: len(r) for name, r in rasters[label].items()}
        finally:
            shutil.rmtree(tmp, ignore_errors=True)
    print("spike counts:", counts, flush=True)
    for p in recurrent.pops:
        assert np.array_equal(rasters["generated"][p.name], rasters["again"][p.name]), f"{p.name}: two runs from one seed differ"
        assert not np.array_equal(rasters["generated"][p.name], rasters["library"][p.name])        # another generator, another matrix
        assert counts["library"][p.name] > 200, counts
        assert abs(counts["generated"][p.name] - counts["library"][p.name]) <= 0.15 * counts["library"][p.name], (p.name, counts)


def test_generated_kernels_regenerate_dense_weights():
    """DENSE connectivity whose weights are never stored but regenerated from their initialisation snippet at every event
    (DENSE_PROCEDURALG; GeNN allows such snippets no random numbers).  Eight sources fire together twice into 500 silent LIF
    neurons through Constant(0.375) weights and a DeltaCurr input: potentials identical, step by step, to the same network with
    StaticPulseConstantWeight."""
    from genn_amd.netspec import Net, Pop, Syn
    n_src, n_trg = 8, 500
    lif = dict(C=1.0, TauM=20.0, Vrest=-60.0, Vreset=-60.0, Vthresh=1e9, Ioffset=0.0, TauRefrac=2.0)

    def potentials(name, **syn):
        net = Net(name=name, dt=1.0, steps=14, seed=777)
        net.pops.append(Pop("S", "ssa", n_src, {}, {"startSpike": (2 * np.arange(n_src)).astype(np.uint32), "endSpike": (2 * np.arange(n_src) + 2).astype(np.uint32)},
                            spike_times=np.tile(np.array([1.0, 11.0], np.float32), n_src)))
        net.pops.append(Pop("T", "lif", n_trg, lif, {"V": np.full(n_trg, -60.0, np.float32), "RefracTime": np.zeros(n_trg, np.float32)}))
        net.syns.append(Syn("ST", "S", "T", matrix="dense", psm="deltacurr", **syn))
        net.snap = 1
        tmp = tempfile.mkdtemp(prefix="adapter_dense_regenerated_")
        try:
            spec, work, out = (os.path.join(tmp, d) for d in ("spec", "work", "out"))
            for d in (work, out):
                os.makedirs(d)
            write_netspec(net, spec)
            print(f"adapter regenerated dense weights ({net.name}): running {DRIVER}", flush=True)
            res = subprocess.run([DRIVER, spec, work, out, "--kernels=generated"], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=240)
            assert res.returncode == 0, res.stdout[-3000:]
            return np.fromfile(os.path.join(out, "T.V.f32"), np.float32).reshape(net.steps, n_trg)
        finally:
            shutil.rmtree(tmp, ignore_errors=True)

    constant = potentials("dense_constant", wum="static", g_init=("Constant", {"constant": 0.375}))
    twin = potentials("dense_twin", wum="static_const", wum_params={"g": 0.375})
    assert np.array_equal(constant, twin)
    moved = [k for k in range(len(constant)) if np.any(constant[k] != np.float32(-60.0))]
    assert moved and np.allclose(constant[moved[0]], -60.0 + (1.0 - np.exp(-1.0 / 20.0)) * 20.0 * n_src * 0.375, rtol=1e-6)


def test_generated_kernels_with_simulation_random_numbers():
    """Random numbers in simulation code (the built-in Poisson neuron, neuronModels.h:307-325: `gennrand_exponential()` refills a
    countdown): the generated kernels draw them from a counter-based generator keyed by the model's seed.  Every backend of
    the reference draws from a generator of its own, so its CPU backend's fixture pins statistics, not spikes: the input
    population's spike count and that of the LIF population it drives agree with the fixture's within sampling error, the
    inter-spike intervals are exponential with the configured mean, neurons are independent, and the same seed gives the same
    raster again."""
    golden = np.load(os.path.join(HERE, "golden", "poisson_input_small.npz"))
    rasters = []
    for attempt in range(2):
        net, snap, tmp, out = _run("poisson_input_small")
        try:
            assert net.generated_kernels
            assert str(golden["input_digest"]) == net.input_digest()
            rasters.append({p.name: np.fromfile(os.path.join(out, f"{p.name}.spikes.u32"), np.uint32).reshape(-1, 2) for p in net.pops})
        finally:
            shutil.rmtree(tmp, ignore_errors=True)
    for name in ("In", "Out"):
        assert np.array_equal(rasters[0][name], rasters[1][name]), f"{name}: the same seed gave another raster"
    got, n_in, steps = rasters[0]["In"], net.pop("In").n, net.steps
    rate_per_step = net.pop("In").params["rate"] * net.dt / 1000.0
    expected = n_in * steps * rate_per_step
    # counts: against the expectation and against the reference backend's draw of the same process (5 sigma of a difference)
    assert abs(len(got) - expected) <= 5.0 * np.sqrt(expected), f"{len(got)} input spikes, expected about {expected:.0f}"
    assert abs(len(got) - len(golden["spikes.In"])) <= 5.0 * np.sqrt(2.0 * expected)
    assert not np.array_equal(got, golden["spikes.In"])                      # (another generator: other spikes)
    # neurons: counts of a renewal process with exponential intervals have variance ~ mean
    counts = np.bincount(got[:, 1], minlength=n_in)
    assert 0.8 <= counts.var() / counts.mean() <= 1.2, f"Fano factor {counts.var() / counts.mean():.3f}"
    # intervals: exponential, so coefficient of variation 1; their mean inside a window of 1,000 steps falls short of
    # 1 / rate = 50 steps (long intervals do not fit), by how much the reference's own raster says
    def intervals(raster):
        order = np.lexsort((raster[:, 0], raster[:, 1]))
        t, i = raster[order, 0].astype(np.float64), raster[order, 1]
        return t, i, np.diff(t)[np.diff(i) == 0]
    t, i, isi = intervals(got)
    ref_isi = intervals(golden["spikes.In"])[2]
    assert 0.9 / rate_per_step <= ref_isi.mean() <= 1.0 / rate_per_step
    assert abs(isi.mean() - ref_isi.mean()) <= 0.02 * ref_isi.mean(), f"mean interval {isi.mean():.2f} steps, the reference's {ref_isi.mean():.2f}"
    assert abs(isi.std() / isi.mean() - 1.0) <= 0.05, f"CV of the intervals {isi.std() / isi.mean():.3f}"
    # no two neurons share a train (streams are per neuron)
    trains = {tuple(t[i == k][:5]) for k in range(0, n_in, 7)}
    assert len(trains) >= 0.99 * len(range(0, n_in, 7))
    # the driven population: same input statistics, same connectivity, so the same output rate up to sampling error
    out_got, out_ref = len(rasters[0]["Out"]), len(golden["spikes.Out"])
    assert out_ref > 2000 and abs(out_got - out_ref) <= 0.05 * out_ref, f"{out_got} output spikes against {out_ref}"


def test_generated_kernels_with_random_numbers_in_weight_update_code():
    """`gennrand_uniform()` in presynaptic spike code (synapses that release with probability 0.4).  No backend of the reference
    pins this — its CPU backend refuses the model ("Undefined identifier" for gennrand_* in weight-update code), its SIMT backends
    each draw from generators of their own — so the check is against what the mathematics fixes: a population whose threshold is
    out of reach integrates its input linearly, so its mean potential must equal that of a twin network with static synapses of
    0.4 times the weight (the expectation); synapses with release probability 1 must reproduce the twin's static projection
    spike for spike; neuron by neuron the stochastic input must differ from its expectation; and the same seed must give
    the same result again."""
    from genn_amd import configs
    results = []
    for twin, repeat in ((False, 0), (False, 1), (True, 0)):
        net = configs.stochastic_synapses(twin=twin)
        net.snap = 100
        tmp = tempfile.mkdtemp(prefix="adapter_stochastic_")
        try:
            spec, work, out = (os.path.join(tmp, d) for d in ("spec", "work", "out"))
            for d in (work, out):
                os.makedirs(d)
            write_netspec(net, spec)
            print(f"adapter stochastic synapses (twin={twin}): running {DRIVER}", flush=True)
            res = subprocess.run([DRIVER, spec, work, out] + (["--kernels=generated"] if twin else []), stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=240)
            assert res.returncode == 0, res.stdout[-3000:]
            code = open(os.path.join(work, net.name + "_CODE", "synapseUpdate.cc")).read()
            assert "__global__" in code and (("gennmi_kernel::rngUniform(gennmiRng)" in code) != twin)
            results.append({"C": np.fromfile(os.path.join(out, "C.spikes.u32"), np.uint32).reshape(-1, 2),
                            "A": np.fromfile(os.path.join(out, "A.spikes.u32"), np.uint32).reshape(-1, 2),
                            "V": np.fromfile(os.path.join(out, "B.V.f32"), np.float32).reshape(net.steps // net.snap, -1)})
        finally:
            shutil.rmtree(tmp, ignore_errors=True)
    first, again, twin = results
    # (the same draws, added up in whatever order the atomics came: equal up to the rounding of reordered sums)
    assert np.allclose(first["V"], again["V"], rtol=1e-5, atol=0.0) and np.array_equal(first["C"], again["C"]), "the same seed gave another result"
    assert len(first["A"]) > 5000 and np.array_equal(first["A"], twin["A"])
    assert len(twin["C"]) > 500 and np.array_equal(first["C"], twin["C"]), "release probability 1 must behave like a static synapse"
    rest = -60.0
    for k in range(first["V"].shape[0]):
        got, want = first["V"][k].astype(np.float64) - rest, twin["V"][k].astype(np.float64) - rest
        assert want.mean() > 0.5
        assert abs(got.mean() - want.mean()) <= 0.02 * want.mean(), f"snapshot {k}: mean depolarisation {got.mean():.4f} against {want.mean():.4f}"
        assert np.abs(got - want).std() > 0.01 * want.mean(), "the stochastic input equals its expectation neuron by neuron"


@pytest.mark.parametrize("config", ["snippet_initialised", "snippet_initialised_layers"])
def test_adapter_device_initialisation_matches_host_layer(config):
    """Preferences::deviceInitialisation through GeNN's generator and Runtime: SPARSE matrices built by FixedProbability
    (with and without autapses) and FixedNumberPostWithReplacement with Uniform, Normal, Constant and constant-parameter
    weights; in the second network by Conv2D with kernel-initialised weights and FixedNumberPreWithReplacement.  The adapter
    numbers the generator streams by projection name, so the Python host layer given the same numbering must produce the very
    same matrices (row lengths, targets, weights) and then the same rasters; with the switch off the reference's host code
    draws from mt19937, which gives other matrices of the same distribution — and, for Conv2D, where nothing is drawn, the
    very same matrix: the reference's own row build code and kernel indexing, run on the host, against the device generator.
    Further runs place the matrices on the device only (VarLocation::DEVICE: nothing is copied back, the rasters must not
    change) and take the step's kernels from generated code."""
    from genn_amd import configs
    from genn_amd.genn_model import model_from_net
    net = configs.snippet_initialised(n_e=1600, n_i=400, steps=150) if config == "snippet_initialised" else configs.snippet_initialised_layers(steps=150)
    net.snap = 0
    tmp = tempfile.mkdtemp(prefix="adapter_devinit_")
    try:
        spec = os.path.join(tmp, "spec")
        write_netspec(net, spec)
        outs = {}
        for flag in (True, False):
            work, out = os.path.join(tmp, f"work{int(flag)}"), os.path.join(tmp, f"out{int(flag)}")
            os.makedirs(work); os.makedirs(out)
            print(f"adapter device initialisation ({flag}): running {DRIVER}", flush=True)
            res = subprocess.run([DRIVER, spec, work, out] + (["--device-init"] if flag else []), stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=240)
            assert res.returncode == 0, res.stdout[-3000:]
            outs[flag] = out
        # (generated kernels only for the first network: the reference's own generic update code cannot print a merged group
        # whose archetype has a kernel size while another member has none — getKernelIndex, codeGenUtils.h:131-151, reads
        # every member's kernel size — and the second network's Conv2D projection merges with a plain SPARSE one)
        variants = [("device arrays", ["--device-init", "--device-arrays"])]
        if config == "snippet_initialised":
            variants.append(("generated", ["--device-init", "--device-arrays", "--kernels=generated"]))
        for label, options in variants:
            work, out = os.path.join(tmp, f"work_{label[:6]}"), os.path.join(tmp, f"out_{label[:6]}")
            os.makedirs(work); os.makedirs(out)
            print(f"adapter device initialisation ({label}): running {DRIVER}", flush=True)
            res = subprocess.run([DRIVER, spec, work, out] + options, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=240)
            assert res.returncode == 0, res.stdout[-3000:]
            assert re.search(r"ready after \S+ s", res.stdout)
            outs[label] = out
        model = model_from_net(net)
        model.load(num_recording_timesteps=net.steps)
        for s in net.syns:
            sg = model.synapse_populations[s.name]
            n_pre = net.pop(s.src).n
            stride = int(open(os.path.join(outs[True], f"{s.name}.rowStride.txt")).read())
            assert stride == sg.row_stride
            got_len = np.fromfile(os.path.join(outs[True], f"{s.name}.rowLength.u32"), np.uint32)
            got_ind = np.fromfile(os.path.join(outs[True], f"{s.name}.ind.u32"), np.uint32).reshape(n_pre, stride)
            want_len = sg.vars["rowLength"].pull_from_device()
            want_ind = sg.vars["ind"].pull_from_device().reshape(n_pre, stride)
            mask = np.arange(stride)[None, :] < want_len[:, None]
            assert np.array_equal(got_len, want_len), f"{s.name}: row lengths differ"
            assert np.array_equal(got_ind[mask], want_ind[mask]), f"{s.name}: targets differ"
            if s.wum != "static_const":
                got_g = np.fromfile(os.path.join(outs[True], f"{s.name}.g.f32"), np.float32).reshape(n_pre, stride)
                assert np.array_equal(got_g[mask], sg.vars["g"].pull_from_device().reshape(n_pre, stride)[mask]), f"{s.name}: weights differ"
            # host initialisation: another draw of the same distribution
            host_len = np.fromfile(os.path.join(outs[False], f"{s.name}.rowLength.u32"), np.uint32)
            assert not np.array_equal(host_len, got_len) or s.connect[0] in ("FixedNumberPostWithReplacement", "Conv2D")
            assert abs(host_len.mean() - got_len.mean()) <= 0.05 * got_len.mean() + 1e-9
            if s.connect[0] == "Conv2D":
                host_ind = np.fromfile(os.path.join(outs[False], f"{s.name}.ind.u32"), np.uint32).reshape(n_pre, stride)
                host_g = np.fromfile(os.path.join(outs[False], f"{s.name}.g.f32"), np.float32).reshape(n_pre, stride)
                assert np.array_equal(host_len, got_len) and np.array_equal(host_ind[mask], got_ind[mask]) and np.array_equal(host_g[mask], got_g[mask])
            if s.connect[0] == "FixedNumberPreWithReplacement":
                for lengths, ind in ((got_len, got_ind), (host_len, np.fromfile(os.path.join(outs[False], f"{s.name}.ind.u32"), np.uint32).reshape(n_pre, stride))):
                    valid = np.arange(stride)[None, :] < lengths[:, None]
                    assert np.all(np.bincount(ind[valid], minlength=net.pop(s.trg).n) == s.connect[1]["num"])
        model.run(net.steps)
        model.pull_recording_buffers_from_device()
        total = 0
        for p in net.pops:
            got = np.fromfile(os.path.join(outs[True], f"{p.name}.spikes.u32"), np.uint32).reshape(-1, 2)
            want = _raster(model, net, p.name)
            assert np.array_equal(got, want), f"raster of {p.name} differs ({len(got)} vs {len(want)} spikes)"
            for label, _ in variants:
                other = np.fromfile(os.path.join(outs[label], f"{p.name}.spikes.u32"), np.uint32).reshape(-1, 2)
                # (generated kernels add a step's inputs in another order: the rasters agree until rounding separates them)
                if label == "generated":
                    first = _first_difference(other, want)
                    assert first is None or first >= 50, f"{label}: raster of {p.name} differs at step {first}"
                else:
                    assert np.array_equal(other, want), f"{label}: raster of {p.name} differs"
            total += len(want)
        assert total > 1000
        model.unload()
    finally:
        shutil.rmtree(tmp, ignore_errors=True)


def _procedural_pair(net, steps, snap):
    """Runs `net` through GeNN's generator and Runtime on the adapter and through the Python host layer with the adapter's
    stream numbering; returns (driver output directory, temporary directory, host-layer model after `steps` steps,
    V and outPost of the host layer after every `snap` steps)."""
    from genn_amd.genn_model import model_from_net
    net.steps, net.snap = steps, snap
    tmp = tempfile.mkdtemp(prefix="adapter_proc_")
    spec, work, out = (os.path.join(tmp, d) for d in ("spec", "work", "out"))
    for d in (work, out):
        os.makedirs(d)
    write_netspec(net, spec)
    print(f"adapter procedural: running {DRIVER}", flush=True)
    res = subprocess.run([DRIVER, spec, work, out], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=240)
    assert res.returncode == 0, res.stdout[-3000:]
    model = model_from_net(net)
    model.load(num_recording_timesteps=steps)
    state = []
    for _ in range(steps // snap):
        for _ in range(snap):
            model.step_time()
        state.append({**{f"V.{p.name}": model.neuron_populations[p.name].vars["V"].pull_from_device().copy() for p in net.pops},
                      **{f"outPost.{s.name}": model.synapse_populations[s.name].vars["outPost"].pull_from_device().copy() for s in net.syns
                         if "outPost" in model.synapse_populations[s.name].vars}})
    model.pull_recording_buffers_from_device()
    return out, tmp, model, state


def test_adapter_dense_kernel_and_neuron_variables_initialised_on_the_device():
    """Preferences::deviceInitialisation for the variables of a stored DENSE matrix, of a TOEPLITZ projection's kernel
    (initGroupMerged.cc:563-593) and of a neuron population (:126-196): with the switch the dumped values are exactly what
    gennmi_init_var draws for the model's seed and the array's stream (2k + 2 for the k-th projection by name, 8000 + 16 p + v
    for variable v of the p-th population by name), and the host loops of those variables are not generated; without it the
    reference's host loops draw other values of the same distribution (Uniform and Normal, Kolmogorov-Smirnov).  Both runs step
    the model afterwards."""
    import ctypes as C
    from scipy import stats
    from genn_amd import _abi, configs, rng
    from genn_amd.genn_model import Array
    from genn_amd.netspec import Net, Pop, Syn
    seed, steps = 91, 40
    net = Net(name="dense_kernel_init", dt=1.0, steps=steps, seed=seed)
    start, end, times = configs.poisson_spike_source(seed, 1, 8 * 8 * 2, 60.0, steps, 1.0)
    net.pops.append(Pop("In", "ssa", 8 * 8 * 2, {}, {"startSpike": start, "endSpike": end}, spike_times=times))
    lif = dict(C=1.0, TauM=20.0, Vrest=-60.0, Vreset=-60.0, Vthresh=-50.0, Ioffset=0.4, TauRefrac=2.0)
    net.pops.append(Pop("Mid", "lif", 8 * 8 * 4, dict(lif), {"V": (-60.0 + 9.0 * rng.uniform(seed, 2, 0, 8 * 8 * 4)).astype(np.float32), "RefracTime": np.zeros(8 * 8 * 4, np.float32)}))
    net.pops.append(Pop("Out", "lif_init", 700, dict(lif, Vmin=-60.0, Vmax=-51.0), {}))
    net.syns.append(Syn("InMid", "In", "Mid", matrix="conv2d", wum="static", psm="expcurr", tau=5.0, g_init=("Normal", {"mean": 0.1, "sd": 0.05}),
                        conv=dict(conv_kh=3, conv_kw=3, conv_ih=8, conv_iw=8, conv_ic=2, conv_oh=8, conv_ow=8, conv_oc=4)))
    net.syns.append(Syn("MidOut", "Mid", "Out", matrix="dense_init", wum="static", psm="expcurr", tau=5.0, g_init=("Uniform", {"min": -0.01, "max": 0.03})))
    net.snap = 0
    tmp = tempfile.mkdtemp(prefix="adapter_dense_init_")
    try:
        spec = os.path.join(tmp, "spec")
        write_netspec(net, spec)
        weights = {}
        for flag in (True, False):
            work, out = os.path.join(tmp, f"work{int(flag)}"), os.path.join(tmp, f"out{int(flag)}")
            os.makedirs(work); os.makedirs(out)
            print(f"adapter dense / kernel initialisation ({flag}): running {DRIVER}", flush=True)
            res = subprocess.run([DRIVER, spec, work, out] + (["--device-init"] if flag else []), stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=240)
            assert res.returncode == 0, res.stdout[-3000:]
            init = open(os.path.join(work, net.name + "_CODE", "init.cc")).read()
            assert init.count("gennmi_init_var(") == (4 if flag else 0)          # two matrices, V and RefracTime (a constant is a snippet too)
            weights[flag] = {s.name: np.fromfile(os.path.join(out, f"{s.name}.g.f32"), np.float32) for s in net.syns}
            weights[flag]["Out.V"] = np.fromfile(os.path.join(out, "Out.V0.f32"), np.float32)
            assert sum(len(np.fromfile(os.path.join(out, f"{p.name}.spikes.u32"), np.uint32)) // 2 for p in net.pops[1:]) > 100
        lib = _abi.load()
        _abi.check(lib.gennmi_init(0))
        place = sorted(p.name for p in net.pops).index("Out")
        for name, stream, count, snippet, params, law in (
                ("InMid", 2, 3 * 3 * 2 * 4, "Normal", (0.1, 0.05), stats.norm(0.1, 0.05)),
                ("MidOut", 4, 256 * 700, "Uniform", (-0.01, 0.03), stats.uniform(-0.01, 0.04)),
                ("Out.V", 8000 + 16 * place, 700, "Uniform", (-60.0, -51.0), stats.uniform(-60.0, 9.0))):
            a = Array(count, np.float32, device_only=True)
            p = (C.c_double * 4)(*(list(params) + [0.0, 0.0]))
            _abi.check(lib.gennmi_init_var(a.ptr, _abi.ELEMENT_TYPES["float32"], count, _abi.INIT_SNIPPETS[snippet], C.byref(p), seed, stream))
            want = a.pull_from_device().copy()
            a.free()
            assert weights[True][name].shape == want.shape
            assert np.array_equal(weights[True][name], want), f"{name}: values are not the device generator's"
            assert not np.array_equal(weights[False][name], want)
            for values in (weights[True][name], weights[False][name]):
                assert stats.kstest(values.astype(np.float64), law.cdf).pvalue > 0.00034, name
    finally:
        shutil.rmtree(tmp, ignore_errors=True)


def test_adapter_zero_copy_recording_buffers():
    """VarLocation::HOST_DEVICE_ZERO_COPY (hip/backend.cc:90-103): with NeuronGroup::setRecordingZeroCopyEnabled the recording
    buffers are pinned host memory mapped into the device's address space — the kernels write the spike words straight into
    them, pulls copy nothing — and the rasters must be those of the reference CPU backend's fixture, on the resident plan with
    its step queue and with every step launched when asked for."""
    net, snap = CASES["va_small"]()
    net.snap = snap
    golden = np.load(os.path.join(HERE, "golden", "va_small.npz"))
    tmp = tempfile.mkdtemp(prefix="adapter_zero_copy_")
    try:
        spec = os.path.join(tmp, "spec")
        write_netspec(net, spec)
        for label, options in (("queued", []), ("eager", ["--step-queue=0"])):
            work, out = os.path.join(tmp, "work_" + label), os.path.join(tmp, "out_" + label)
            os.makedirs(work); os.makedirs(out)
            print(f"adapter zero-copy recording ({label}): running {DRIVER}", flush=True)
            res = subprocess.run([DRIVER, spec, work, out, "--zero-copy-recording"] + options, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=240)
            assert res.returncode == 0, res.stdout[-3000:]
            for p in net.pops:
                got = np.fromfile(os.path.join(out, f"{p.name}.spikes.u32"), np.uint32).reshape(-1, 2)
                assert np.array_equal(got, golden[f"spikes.{p.name}"]), f"{label}: raster of {p.name} differs"
    finally:
        shutil.rmtree(tmp, ignore_errors=True)


def _first_difference(a, b):
    """First timestep at which two rasters ((step, neuron) pairs in ascending order) differ, or None."""
    if np.array_equal(a, b):
        return None
    n = min(len(a), len(b))
    diff = np.nonzero(np.any(a[:n] != b[:n], axis=1))[0]
    k = int(diff[0]) if len(diff) else n
    return int(min(a[k, 0] if k < len(a) else 1 << 30, b[k, 0] if k < len(b) else 1 << 30))


def _raster(model, net, name):
    times, ids = model.neuron_populations[name].spike_recording_data[0]
    return np.stack([np.rint(times / net.dt).astype(np.uint32), ids.astype(np.uint32)], axis=1)


def test_adapter_procedural_matches_host_layer():
    """A model with PROCEDURAL projections through GeNN's generator and Runtime on the adapter against the same network
    through the Python host layer with the adapter's stream numbering: both must regenerate the same matrices and weights
    from the seed.  (The reference's own backends draw procedural rows from their own generators, so there is no reference
    fixture for this path; the regenerated matrix is held to the stored one by tests/test_gpu_procedural.py and to the
    snippets' distributions by tests/test_gpu_init.py.)

    Uniform and Normal weights: accumulators and V after each of the first six steps within 1e-5 (had a stream, a parameter
    or a row differed, they would differ in the first digit), rasters identical.  One dyadic weight per projection into
    DeltaCurr inputs — sums exact in any atomic order: rasters and V identical over 100 steps."""
    from genn_amd import configs
    net = configs.procedural()
    out, tmp, model, state = _procedural_pair(net, steps=6, snap=1)
    try:
        spikes = 0
        for p in net.pops:
            got = np.fromfile(os.path.join(out, f"{p.name}.spikes.u32"), np.uint32).reshape(-1, 2)
            assert np.array_equal(got, _raster(model, net, p.name)), f"raster of {p.name} differs"
            spikes += len(got)
            v = np.fromfile(os.path.join(out, f"{p.name}.V.f32"), np.float32).reshape(6, p.n)
            for k in range(6):
                _close(v[k], state[k][f"V.{p.name}"], f"V of {p.name} after step {k}")
        for s in net.syns:
            acc = np.fromfile(os.path.join(out, f"{s.name}.outPost.f32"), np.float32).reshape(6, -1)
            for k in range(6):
                _close(acc[k], state[k][f"outPost.{s.name}"], f"outPost of {s.name} after step {k}", accumulator=True)
            assert np.abs(acc).max() > 0.05
        assert spikes > 50
        model.unload()
    finally:
        shutil.rmtree(tmp, ignore_errors=True)

    net = configs.procedural(order_free=True)
    out, tmp, model, state = _procedural_pair(net, steps=100, snap=50)
    try:
        spikes = 0
        for p in net.pops:
            got = np.fromfile(os.path.join(out, f"{p.name}.spikes.u32"), np.uint32).reshape(-1, 2)
            assert np.array_equal(got, _raster(model, net, p.name)), f"raster of {p.name} differs"
            spikes += len(got)
            v = np.fromfile(os.path.join(out, f"{p.name}.V.f32"), np.float32).reshape(2, p.n)
            for k in range(2):
                assert np.array_equal(v[k], state[k][f"V.{p.name}"]), f"V of {p.name} after {50 * (k + 1)} steps"
        assert spikes > 2000
        model.unload()
    finally:
        shutil.rmtree(tmp, ignore_errors=True)


def test_adapter_poisson_background_matches_host_layer():
    """The scaled cortical microcircuit with PoissonExp current sources through GeNN's generator and Runtime on the adapter
    against the same network through the Python host layer: the adapter must number the sources' generator streams, pass
    the model's seed and round the derived parameters (ExpDecay, Init, ExpMinusLambda: currentSourceModels.h:123-128) so
    that both draw the same numbers — rasters identical over 40 ms, V within 1e-5.  (The
    reference's backends draw this background from their own generators; the statistics are held to the reference's CPU
    backend by tests/test_gpu_poisson.py.)"""
    from genn_amd import configs
    net = configs.potjans(neuron_scale=0.05, connectivity_scale=0.2, steps=400, poisson=True)
    out, tmp, model, state = _procedural_pair(net, steps=400, snap=200)
    try:
        spikes = 0
        for p in net.pops:
            got = np.fromfile(os.path.join(out, f"{p.name}.spikes.u32"), np.uint32).reshape(-1, 2)
            assert np.array_equal(got, _raster(model, net, p.name)), f"raster of {p.name} differs"
            spikes += len(got)
            v = np.fromfile(os.path.join(out, f"{p.name}.V.f32"), np.float32).reshape(2, p.n)
            for k in range(2):
                _close(v[k], state[k][f"V.{p.name}"], f"V of {p.name} after {200 * (k + 1)} steps")
        assert spikes > 300
        model.unload()
    finally:
        shutil.rmtree(tmp, ignore_errors=True)


def test_genn_buildmodel_flow_matches_the_reference_backend():
    """The reference's own generator driver (src/genn/generator/generator.cc, built by oracle/Makefile.ref with
    -DBACKEND_NAMESPACE=MI355X as genn_amd/backend/MakefileMI355X sets it) on the example model file
    genn_amd/backend/example/model.cc: generate, compile, construct the Runtime, and run the model file's simulate() — 3000
    steps of the balanced network, connectivity and initial state from GeNN's seeded built-in snippets.  Spike counts and
    raster checksums must equal what the same driver built for the SingleThreadedCPU backend printed
    (tests/golden/selection_example.json, written by tests/golden/make_selection_golden.py)."""
    import json
    import re
    generator = os.path.join(ROOT, "oracle", "_ref", "mi355x_generator")
    if not os.path.exists(generator):
        pytest.skip("oracle/_ref/mi355x_generator is not built")
    golden = json.load(open(os.path.join(HERE, "golden", "selection_example.json")))
    tmp = tempfile.mkdtemp(prefix="buildmodel_")
    try:
        res = subprocess.run([generator, ROOT, tmp, "1"], cwd=tmp, env=dict(os.environ, GENN_EXAMPLE_STEPS=str(golden["steps"])),
                             stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=300)
        assert res.returncode == 0, res.stdout[-3000:]
        got = {m.group(1): {"spikes": int(m.group(2)), "checksum": m.group(3)}
               for m in re.finditer(r"example: population (\w+) spikes (\d+) checksum (\d+)", res.stdout)}
        assert got == golden["populations"], (got, golden["populations"])
    finally:
        shutil.rmtree(tmp, ignore_errors=True)
