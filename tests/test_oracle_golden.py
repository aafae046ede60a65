"""CPU tests that pin the oracle (oracle/genn_cpu.c).

1. Golden vectors written by the reference's own SingleThreadedCPU backend (tests/golden/*.npz,
   made by tests/golden/make_golden.py): spike rasters, state snapshots, plastic weights and the
   column remap must match bit for bit.
2. The closed-form answers of the reference's feature tests (tests/features/test_event_propagation.py)
   and its Toeplitz fixtures.
3. What the mathematics fixes: LIF exact integration, trace-STDP weight changes of isolated pairs,
   dense matrix-vector products on tiny inputs.
"""
import math
import os
import sys

import numpy as np
import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(HERE, "golden"))

from cases import CASES, REFERENCE_ONLY  # noqa: E402
from genn_amd.netspec import Net, Pop, Syn, CurrentSource  # noqa: E402
from oracle.genn_cpu import OracleNet, literal_f32  # noqa: E402

FIXTURES = os.path.join(HERE, "golden", "reference_fixtures")


@pytest.mark.parametrize("case", sorted(set(CASES) - REFERENCE_ONLY))
def test_oracle_matches_reference_backend(case):
    gold = np.load(os.path.join(HERE, "golden", case + ".npz"))
    net, snap = CASES[case]()
    assert net.input_digest() == str(gold["input_digest"]), "the input generator no longer reproduces the golden inputs"
    fuse = dict(item.split("=") for item in gold["fusemap"].tolist())
    col = {s.name: int(gold[f"colStride.{s.name}"]) for s in net.syns if f"colStride.{s.name}" in gold}
    record_events = [s.name for s in net.syns if f"events.{s.name}" in gold]
    oracle = OracleNet(net, num_recording_timesteps=net.steps if record_events else 0, col_stride=col or None)
    for s in net.syns:
        if s.name in col:
            col_length = gold[f"colLength.{s.name}"]
            assert np.array_equal(oracle.col_length(s.name), col_length)
            mask = np.arange(col[s.name])[None, :] < col_length[:, None]
            assert np.array_equal(oracle.remap(s.name).reshape(-1, col[s.name])[mask], gold[f"remap.{s.name}"].reshape(-1, col[s.name])[mask])
    raster = {p.name: [] for p in net.pops}
    k = 0
    for step in range(net.steps):
        oracle.step()
        for p in net.pops:
            ids = oracle.spikes(p.name)
            assert np.all(np.diff(ids.astype(np.int64)) > 0), "spike queue must be in ascending neuron order"
            raster[p.name].append(np.stack([np.full(len(ids), step, np.uint32), ids], axis=1))
        if (step + 1) % snap == 0:
            for p in net.pops:
                names = {"lif": ("V", "RefracTime"), "izh": ("V", "U"), "ssa": ()}[p.model]
                for which, name in enumerate(names):
                    assert np.array_equal(oracle.var(p.name, which), gold[f"{name}.{p.name}"][k]), f"{name}.{p.name} at step {step}"
            for s in net.syns:
                if fuse[s.name] == s.name:
                    assert np.array_equal(oracle.out_post(s.name), gold[f"outPost.{s.name}"][k]), f"outPost.{s.name} at step {step}"
                if s.wum == "stdp_trace":
                    assert np.array_equal(oracle.pre_trace(s.src), gold[f"preTrace.{s.name}"][k])
                    assert np.array_equal(oracle.post_trace(s.trg), gold[f"postTrace.{s.name}"][k])
            k += 1
    for s in net.syns:
        if s.wum in ("stdp_trace", "stdp_additive"):
            assert np.array_equal(oracle.syn_g(s.name), gold[f"g.{s.name}"])
            assert np.count_nonzero(gold[f"g.{s.name}"] != s.g.reshape(-1)) > 100, "the fixture's run changed no weight" 
        if fuse[s.name] == s.name and f"denDelay.{s.name}" in gold:
            assert np.array_equal(oracle.den_delay(s.name), gold[f"denDelay.{s.name}"])
    for name in record_events:
        n = net.pop(net.syn(name).src).n
        bits = np.unpackbits(oracle.event_record(name, net.steps).reshape(net.steps, -1).view(np.uint8), axis=1, bitorder="little")[:, :n]
        steps, ids = np.nonzero(bits)
        assert np.array_equal(np.stack([steps, ids], axis=1).astype(np.uint32), gold[f"events.{name}"]), f"recorded events of {name}"
        assert len(steps) > 100
    total = 0
    for p in net.pops:
        mine = np.concatenate(raster[p.name])
        assert np.array_equal(mine, gold[f"spikes.{p.name}"]), f"raster of {p.name}"
        total += len(mine)
    assert total > 100
    oracle.close()


# constants as the reference prints them into generated code (observed in code its CPU backend generated
# for dt = 0.1 and dt = 1 models): double -> "%.9e" -> float
@pytest.mark.parametrize("value,text", [
    (math.exp(-0.1 / 20.0), "9.950124792e-01"), (math.exp(-0.1 / 10.0), "9.900498337e-01"), (math.exp(-0.1 / 5.0), "9.801986733e-01"),
    ((5.0 * (1.0 - math.exp(-0.1 / 5.0))) * (1.0 / 0.1), "9.900663347e-01"), ((10.0 * (1.0 - math.exp(-0.1 / 10.0))) * (1.0 / 0.1), "9.950166251e-01"),
    (math.exp(-0.1 / 0.5), "8.187307531e-01"), ((0.5 * (1.0 - math.exp(-0.1 / 0.5))) * (1.0 / 0.1), "9.063462346e-01"),
    (math.exp(-1.0 / 20.0), "9.512294245e-01"), (math.exp(-1.0 / 10.0), "9.048374180e-01"), (0.55, "5.500000000e-01"), (0.1, "1.000000000e-01")])
def test_literal_rounding_known_answers(value, text):
    assert "%.9e" % value == text
    assert literal_f32(value) == np.float32(text)


def _silent(name, n):
    lif = dict(C=1.0, TauM=20.0, Vrest=-60.0, Vreset=-60.0, Vthresh=1e9, Ioffset=0.0, TauRefrac=5.0)
    return Pop(name, "lif", n, lif, {"V": np.full(n, -60.0, np.float32), "RefracTime": np.zeros(n, np.float32)})


def _one_hot_source(name, n):
    return Pop(name, "ssa", n, {}, {"startSpike": np.arange(n, dtype=np.uint32), "endSpike": np.arange(1, n + 1, dtype=np.uint32)},
               spike_times=np.arange(n, dtype=np.float32))


def _ragged(n_pre, pre, post, values=None, dtype=np.float32):
    order = np.lexsort((post, pre))
    pre, post = np.asarray(pre)[order], np.asarray(post)[order]
    rl = np.bincount(pre, minlength=n_pre).astype(np.uint32)
    stride = max(1, int(rl.max()))
    starts = np.concatenate(([0], np.cumsum(rl)[:-1])).astype(np.int64)
    within = np.arange(len(pre)) - starts[pre]
    ind = np.zeros((n_pre, stride), np.uint32)
    ind[pre, within] = post
    out = None
    if values is not None:
        out = np.zeros((n_pre, stride), dtype)
        out[pre, within] = np.asarray(values)[order]
    return rl, ind, out


# tests/features/test_event_propagation.py:65-260 — decode table
def test_oracle_forward_decode():
    pre, post = zip(*[(i, j) for i in range(16) for j in range(4) if (i + 1) & (1 << j)])
    rl, ind, g = _ragged(16, pre, post, np.ones(len(pre)))
    net = Net("fwd", dt=1.0, steps=16, pops=[_one_hot_source("S", 16), _silent("P", 4)])
    net.syns.append(Syn("SP", "S", "P", wum="static", psm="deltacurr", row_stride=ind.shape[1], row_length=rl, ind=ind, g=g))
    o = OracleNet(net)
    place = 2 ** np.arange(4)
    for step in range(16):
        # observe Isyn of this step: outPost after the synapse update, before the neuron update clears it
        o.l.gc_update_synapses(o.h, np.float32(step))
        value = int(np.sum(place[np.isclose(o.out_post("SP"), 1.0)]))
        assert value == step
        o.l.gc_update_neurons(o.h, np.float32(step), 0)
        o.l.gc_advance(o.h)


# tests/features/test_event_propagation.py:262-329 — dendritic delays 9..0 must deliver exactly 10.0 in step 11
def test_oracle_dendritic_delay_ramp():
    rl, ind, d = _ragged(10, np.arange(10), np.zeros(10, int), np.arange(9, -1, -1), np.uint8)
    net = Net("dd", dt=1.0, steps=12, pops=[_one_hot_source("S", 10), _silent("P", 1)])
    net.syns.append(Syn("SP", "S", "P", wum="static_delay", psm="deltacurr", row_stride=1, row_length=rl, ind=ind,
                        g=np.ones((10, 1), np.float32), d=d, max_den_delay=10))
    o = OracleNet(net)
    for step in range(11):
        o.l.gc_update_synapses(o.h, np.float32(step))
        ring = o.den_delay("SP").reshape(10, 1)
        front = ring[o.l.gc_den_delay_ptr(o.h, o.pop_id["P"], 0), 0]
        assert front == (10.0 if step == 10 else 0.0)
        o.l.gc_update_neurons(o.h, np.float32(step), 0)
        o.l.gc_advance(o.h)


# tests/features/test_event_propagation.py:387-485 with the reference's own Sobel fixtures; also a library routine
def test_oracle_toeplitz_fixtures():
    from scipy.signal import correlate2d
    pattern = np.load(os.path.join(FIXTURES, "test_pattern.npy"))
    end = np.cumsum(np.bincount(pattern, minlength=64 * 64)).astype(np.uint32)
    start = np.concatenate(([0], end[:-1])).astype(np.uint32)
    kernels = {"horizontal": np.asarray([[1.0, 2.0, 1.0], [0.0, 0.0, 0.0], [-1.0, -2.0, -1.0]]),
               "vertical": np.asarray([[1.0, 0.0, -1.0], [2.0, 0.0, -2.0], [1.0, 0.0, -1.0]])}
    conv = dict(conv_kh=3, conv_kw=3, conv_ih=64, conv_iw=64, conv_ic=1, conv_oh=62, conv_ow=62, conv_oc=1)
    image = np.zeros(64 * 64)
    image[pattern] = 1.0
    for name, kern in kernels.items():
        net = Net("toep", dt=1.0, steps=2)
        net.pops.append(Pop("S", "ssa", 64 * 64, {}, {"startSpike": start, "endSpike": end}, spike_times=np.zeros(len(pattern), np.float32)))
        net.pops.append(_silent("P", 62 * 62))
        net.syns.append(Syn("SP", "S", "P", matrix="conv2d", wum="static", psm="deltacurr", g=kern.astype(np.float32).reshape(3, 3, 1, 1), conv=conv))
        o = OracleNet(net)
        o.step()
        o.l.gc_update_synapses(o.h, np.float32(1.0))
        got = o.out_post("SP").copy()
        assert np.allclose(got, np.load(os.path.join(FIXTURES, name + "_output.npy")))
        # the kernel flip inside the Toeplitz snippet cancels the scatter direction: in image coordinates the
        # layer is the plain cross-correlation of the spike image with the kernel
        assert np.allclose(got.reshape(62, 62), correlate2d(image.reshape(64, 64), kern, mode="valid"))


def test_oracle_lif_closed_form():
    """Between spikes LIF is the exact-integration recurrence; with constant input V(k) has a closed form."""
    n = 4
    lif = dict(C=1.0, TauM=20.0, Vrest=-60.0, Vreset=-60.0, Vthresh=-50.0, Ioffset=0.4, TauRefrac=5.0)
    net = Net("lif", dt=0.1, steps=200, pops=[Pop("A", "lif", n, lif, {"V": np.array([-60, -58, -55, -52], np.float32), "RefracTime": np.zeros(n, np.float32)})])
    o = OracleNet(net)
    v0 = o.var("A", 0).astype(np.float64).copy()
    o.run(200)
    v_inf = -60.0 + 0.4 * 20.0
    want = v_inf - (v_inf - v0) * math.exp(-200 * 0.1 / 20.0)
    assert np.allclose(o.var("A", 0), want, rtol=0, atol=2e-4)     # -52 mV is the asymptote: nobody spikes
    # above threshold: spike when V crosses -50, reset, 5 ms (50 steps) refractory
    lif["Ioffset"] = 0.6
    net = Net("lif2", dt=0.1, steps=700, pops=[Pop("A", "lif", 1, lif, {"V": np.array([-51.0], np.float32), "RefracTime": np.zeros(1, np.float32)})])
    o = OracleNet(net)
    spikes = []
    for step in range(700):
        o.step()
        if len(o.spikes("A")):
            spikes.append(step)
    v_inf = -60.0 + 0.6 * 20.0
    first = math.ceil(20.0 / 0.1 * math.log((v_inf + 51.0) / (v_inf + 50.0)))
    assert spikes[0] in (first - 1, first)
    # after a spike: ~50 refractory steps (fp32 countdown from 5.0 in steps of 0.1f), then the charge time from reset
    charge = 20.0 / 0.1 * math.log((v_inf + 60.0) / (v_inf + 50.0))
    assert abs((spikes[1] - spikes[0]) - (50 + charge)) <= 2


def test_oracle_stdp_pair_closed_form():
    """One plastic synapse pre->post driven by two spike sources: a pre spike arriving dT after a post spike
    depresses by aMinus*exp(-dT/tauMinus) (the post trace), a post spike after a pre spike potentiates by
    aPlus*exp(-dT/tauPlus); weights clip to [wMin, wMax]."""
    stdp = dict(tauPlus=20.0, tauMinus=20.0, aPlus=0.01, aMinus=0.012, wMin=0.0, wMax=1.0)
    for pre_t, post_t in ((10.0, 15.0), (15.0, 10.0)):
        pre = Pop("Pre", "ssa", 1, {}, {"startSpike": np.zeros(1, np.uint32), "endSpike": np.ones(1, np.uint32)}, spike_times=np.array([pre_t], np.float32))
        post = Pop("Post", "ssa", 1, {}, {"startSpike": np.zeros(1, np.uint32), "endSpike": np.ones(1, np.uint32)}, spike_times=np.array([post_t], np.float32))
        net = Net("pair", dt=1.0, steps=40, pops=[pre, post])
        net.syns.append(Syn("S", "Pre", "Post", wum="stdp_trace", wum_params=stdp, psm="deltacurr", row_stride=1,
                            row_length=np.ones(1, np.uint32), ind=np.zeros((1, 1), np.uint32), g=np.full((1, 1), 0.5, np.float32)))
        o = OracleNet(net)
        o.run(40)
        g = float(o.syn_g("S")[0])
        dT = abs(post_t - pre_t)
        # the trace seen by the later spike's synapse code has decayed dT times since its bump
        # (the update runs one step after the spike, when the partner's trace has decayed once more and been
        #  bumped one step earlier: net dT decays)
        if post_t > pre_t:
            assert g == pytest.approx(0.5 + 0.01 * math.exp(-dT / 20.0), rel=1e-5)
        else:
            assert g == pytest.approx(0.5 - 0.012 * math.exp(-dT / 20.0), rel=1e-5)
    # clipping
    net.syns[0].g = np.full((1, 1), 0.001, np.float32)
    o = OracleNet(net)
    o.run(40)
    assert float(o.syn_g("S")[0]) == 0.0


def test_oracle_propagation_equals_dense_product():
    """Brute force on tiny inputs: one step of propagation equals W^T s for the 0/1 spike vector."""
    rng = np.random.default_rng(3)
    n_pre, n_post = 23, 17
    dense = np.where(rng.random((n_pre, n_post)) < 0.3, rng.integers(1, 9, (n_pre, n_post)), 0).astype(np.float32)   # small integers: sums exact
    pre, post = np.nonzero(dense)
    rl, ind, g = _ragged(n_pre, pre, post, dense[pre, post])
    fire = rng.random(n_pre) < 0.5
    end = np.cumsum(fire).astype(np.uint32)
    start = (end - fire).astype(np.uint32)
    net = Net("dense", dt=1.0, steps=2)
    net.pops.append(Pop("S", "ssa", n_pre, {}, {"startSpike": start, "endSpike": end}, spike_times=np.zeros(int(fire.sum()), np.float32)))
    net.pops.append(_silent("P", n_post))
    net.syns.append(Syn("SP", "S", "P", wum="static", psm="deltacurr", row_stride=ind.shape[1], row_length=rl, ind=ind, g=g))
    o = OracleNet(net)
    o.step()
    assert np.array_equal(o.spikes("S"), np.flatnonzero(fire))
    o.l.gc_update_synapses(o.h, np.float32(1.0))
    assert np.array_equal(o.out_post("SP"), dense.T @ fire.astype(np.float32))


def _bitmask_words(n_pre, n_post, pre, post):
    """BITMASK connectivity words: bit idPre*rowStride + idPost (row stride = numPost padded to 32), most significant bit
    of a word first (single_threaded_cpu/backend.cc:1393-1404, 2003-2006)."""
    stride = (n_post + 31) // 32 * 32
    bits = np.zeros(n_pre * stride, np.uint8)
    bits[np.asarray(pre) * stride + np.asarray(post)] = 1
    return np.packbits(bits, bitorder="big").view(">u4").astype(np.uint32), stride


# tests/features/test_event_propagation.py:65-260 — the decode table holds for the DENSE, BITMASK and constant-weight
# projections of that test too
@pytest.mark.parametrize("kind", ["dense", "dense_const_all", "bitmask", "sparse_const"])
def test_oracle_forward_decode_other_matrix_types(kind):
    pre, post = map(np.asarray, zip(*[(i, j) for i in range(16) for j in range(4) if (i + 1) & (1 << j)]))
    net = Net("fwd", dt=1.0, steps=16, pops=[_one_hot_source("S", 16), _silent("P", 4)])
    if kind == "dense":
        g = np.zeros((16, 4), np.float32)
        g[pre, post] = 1.0
        net.syns.append(Syn("SP", "S", "P", matrix="dense", wum="static", psm="deltacurr", g=g))
    elif kind == "dense_const_all":
        net.syns.append(Syn("SP", "S", "P", matrix="dense", wum="static_const", wum_params={"g": 1.0}, psm="deltacurr"))
    elif kind == "bitmask":
        gp, stride = _bitmask_words(16, 4, pre, post)
        net.syns.append(Syn("SP", "S", "P", matrix="bitmask", wum="static_const", wum_params={"g": 1.0}, psm="deltacurr", gp=gp, row_stride=stride))
    else:
        rl, ind, _ = _ragged(16, pre, post)
        net.syns.append(Syn("SP", "S", "P", wum="static_const", wum_params={"g": 1.0}, psm="deltacurr", row_stride=ind.shape[1], row_length=rl, ind=ind))
    o = OracleNet(net)
    place = 2 ** np.arange(4)
    for step in range(16):
        o.l.gc_update_synapses(o.h, np.float32(step))
        value = int(np.sum(place[np.isclose(o.out_post("SP"), 1.0)]))
        assert value == (15 if kind == "dense_const_all" and step > 0 else step)
        o.l.gc_update_neurons(o.h, np.float32(step), 0)
        o.l.gc_advance(o.h)


def test_oracle_dense_and_bitmask_equal_matrix_products():
    """Brute force: one step through a DENSE matrix is W^T s, through a BITMASK one g * B^T s (small integers: sums exact)."""
    rng = np.random.default_rng(5)
    n_pre, n_post = 41, 37                      # more than one connectivity word per row, with padding bits
    dense = rng.integers(-4, 5, (n_pre, n_post)).astype(np.float32)
    mask = rng.random((n_pre, n_post)) < 0.4
    fire = rng.random(n_pre) < 0.5
    end = np.cumsum(fire).astype(np.uint32)
    start = (end - fire).astype(np.uint32)
    gp, stride = _bitmask_words(n_pre, n_post, *np.nonzero(mask))
    net = Net("dense", dt=1.0, steps=2)
    net.pops.append(Pop("S", "ssa", n_pre, {}, {"startSpike": start, "endSpike": end}, spike_times=np.zeros(int(fire.sum()), np.float32)))
    net.pops += [_silent("P", n_post), _silent("Q", n_post)]
    net.syns.append(Syn("SP", "S", "P", matrix="dense", wum="static", psm="deltacurr", g=dense))
    net.syns.append(Syn("SQ", "S", "Q", matrix="bitmask", wum="static_const", wum_params={"g": 3.0}, psm="deltacurr", gp=gp, row_stride=stride))
    o = OracleNet(net)
    o.step()
    o.l.gc_update_synapses(o.h, np.float32(1.0))
    assert np.array_equal(o.out_post("SP"), dense.T @ fire.astype(np.float32))
    assert np.array_equal(o.out_post("SQ"), 3.0 * (mask.T.astype(np.float32) @ fire.astype(np.float32)))


def test_oracle_recording_bitfield():
    n = 70
    fire_at = np.arange(n) % 7
    pop = Pop("S", "ssa", n, {}, {"startSpike": np.arange(n, dtype=np.uint32), "endSpike": np.arange(1, n + 1, dtype=np.uint32)},
              spike_times=fire_at.astype(np.float32))
    o = OracleNet(Net("rec", dt=1.0, steps=7, pops=[pop]), num_recording_timesteps=7)
    o.run(7)
    words = (n + 31) // 32
    rec = o.record("S", 7).reshape(7, words)
    bits = np.unpackbits(rec.view(np.uint8), axis=1, bitorder="little")[:, :n]
    assert np.array_equal(bits, (fire_at[None, :] == np.arange(7)[:, None]).astype(np.uint8))


# ---- PoissonExp current source ------------------------------------------------------------------------------------------
def test_oracle_philox_known_answers():
    """The generator under the oracle's PoissonExp source against the published Philox4x32-10 vectors."""
    import ctypes as C
    from oracle import genn_cpu
    from philox_ref import KNOWN_ANSWERS
    lib = genn_cpu.lib()
    for counter, key, want in KNOWN_ANSWERS:
        out = (C.c_uint32 * 4)()
        lib.gc_philox4x32(*counter, *key, C.byref(out))
        assert tuple(out) == want


def _poisson_only(n, weight, tau, rate, dt=0.1, seed=77):
    net = Net(name="poisson_only", dt=dt, steps=100, seed=seed)
    net.pops.append(Pop("P", "lif", n, dict(C=0.25, TauM=10.0, Vrest=-65.0, Vreset=-65.0, Vthresh=1.0e6, Ioffset=0.0, TauRefrac=2.0),
                        {"V": np.full(n, -65.0, np.float32), "RefracTime": np.zeros(n, np.float32)}))
    net.css.append(CurrentSource("P_bg", "poisson_exp", "P", params=dict(weight=weight, tauSyn=tau, rate=rate)))
    return net


def test_oracle_poisson_exp_is_the_snippets_loop():
    """The snippet (currentSourceModels.h:107-122) restated here in numpy from the same generator words: numSpikes is the
    number of uniforms drawn until their running product is no longer above ExpMinusLambda; the state gains
    Init * (numSpikes - 1), is injected, then decays.  One step from zero state leaves current = Init * k * ExpDecay, so
    the counts can be read back from the oracle and compared draw for draw."""
    from philox_ref import philox4x32
    n, weight, tau, rate, dt, seed = 400, 0.0878, 0.5, 30000.0, 0.1, 77
    net = _poisson_only(n, weight, tau, rate, dt, seed)
    o = OracleNet(net)
    o.step()
    decay = np.float32(literal_f32(math.exp(-dt / tau)))
    init = np.float32(literal_f32(weight * (1.0 - math.exp(-dt / tau)) * (tau / dt)))
    lam = np.float32(literal_f32(math.exp(-(rate / 1000.0) * dt)))
    counts = np.zeros(n, np.int64)
    for i in range(n):
        prod, k, call, done = np.float32(1.0), 0, 0, False
        while not done:
            words = philox4x32(i, 0, call, 1000, seed & 0xFFFFFFFF, seed >> 32)
            for w in words:
                k += 1
                prod = np.float32(prod * (np.float32(int(w) >> 8) * np.float32(1.0 / 16777216.0)))
                if not prod > lam:
                    done = True
                    break
            call += 1
        counts[i] = k - 1
    want = (init * counts.astype(np.float32)) * decay
    assert np.array_equal(o.cs_current("P_bg"), want)
    assert counts.max() >= 8                     # some neurons needed a second generator call
    # Poisson counts: mean and variance both lambda = 3
    assert abs(counts.mean() - 3.0) < 5.0 * math.sqrt(3.0 / n) and abs(counts.var() - 3.0) < 1.0


def test_oracle_poisson_exp_stationary_moments():
    """Shot noise with kernel Init * a^k, a = exp(-dt / tau): the injected value has mean Init * lambda / (1 - a) (which is
    weight * tau * rate, the mean the snippet's Init is chosen for) and variance Init^2 * lambda / (1 - a^2)."""
    weight, tau, rate, dt, n = 0.0878, 0.5, 12800.0, 0.1, 40000
    o = OracleNet(_poisson_only(n, weight, tau, rate, dt))
    o.run(60)
    a = math.exp(-dt / tau)
    init = weight * (1.0 - a) * (tau / dt)
    lam = rate / 1000.0 * dt
    got = o.cs_current("P_bg").astype(np.float64) / a
    mean, var = init * lam / (1.0 - a), init * init * lam / (1.0 - a * a)
    assert abs(mean - weight * tau * rate / 1000.0) < 1e-12
    assert abs(got.mean() - mean) < 5.0 * math.sqrt(var / n)
    assert abs(got.var() - var) < 0.05 * var
