"""Synthetic-input generators for the benchmark configurations (and reduced-scale twins).

Every array comes from the repo's counter-based generator (:mod:`genn_amd.rng` for small
arrays, :mod:`genn_amd.netgen` — the same streams, multi-threaded C — for per-synapse ones); a
(config, scale, seed) triple therefore names one exact network.  Rows are sorted by
postsynaptic index, as the reference's built-in connectivity snippets and
``set_sparse_connections`` produce them (pygenn/genn_groups.py:447-460).
"""
import math

import numpy as np

from . import netgen, rng
from .netspec import Net, Pop, CurrentSource, Syn, Custom


def _const_rows(row_length, stride, value):
    return np.where(np.arange(stride)[None, :] < row_length[:, None], np.float32(value), np.float32(0)).astype(np.float32)


# --------------------------------------------------------------------------------------------
# C1: balanced LIF network (Vogels-Abbott shape)
# --------------------------------------------------------------------------------------------
def vogels_abbott(n=4000, steps=10000, seed=1234, p=0.02, dt=0.1, ioffset=0.55, pad=1, axonal_delays=None):
    """Balanced LIF network (E/I 4:1, fixed connection probability).  `axonal_delays`: axonal delay in timesteps per
    projection name ("EE", "EI", "IE", "II"), default none."""
    n_e = (n * 4) // 5
    n_i = n - n_e
    lif = dict(C=1.0, TauM=20.0, Vrest=-60.0, Vreset=-60.0, Vthresh=-50.0, Ioffset=ioffset, TauRefrac=5.0)
    net = Net(name="va", dt=dt, steps=steps, seed=seed)
    for k, (name, num) in enumerate((("E", n_e), ("I", n_i))):
        v0 = (-60.0 + 10.0 * rng.uniform(seed, 1 + k, 0, num)).astype(np.float32)
        net.pops.append(Pop(name, "lif", num, dict(lif), {"V": v0, "RefracTime": np.zeros(num, np.float32)}))
    stream = 16
    for src, n_src, w, tau in (("E", n_e, 0.5, 5.0), ("I", n_i, -2.25, 10.0)):
        for trg, n_trg in (("E", n_e), ("I", n_i)):
            rl, ind = netgen.fixed_probability(seed, stream, n_src, n_trg, p, pad=pad)
            stream += 1
            net.syns.append(Syn(f"{src}{trg}", src, trg, wum="static", psm="expcurr", tau=tau,
                                row_stride=ind.shape[1], row_length=rl, ind=ind, g=_const_rows(rl, ind.shape[1], w),
                                axonal_delay_steps=int((axonal_delays or {}).get(f"{src}{trg}", 0))))
    return net


# --------------------------------------------------------------------------------------------
# C2: Potjans-Diesmann cortical microcircuit (constants: userproject/potjans_microcircuit.py:27-100)
# --------------------------------------------------------------------------------------------
PD_LAYERS = ("23", "4", "5", "6")
PD_NUM = {"23E": 20683, "23I": 5834, "4E": 21915, "4I": 5479, "5E": 4850, "5I": 1065, "6E": 14395, "6I": 2948}
PD_PROB = {  # [target][source]
    "23E": {"23E": 0.1009, "23I": 0.1689, "4E": 0.0437, "4I": 0.0818, "5E": 0.0323, "5I": 0.0, "6E": 0.0076, "6I": 0.0},
    "23I": {"23E": 0.1346, "23I": 0.1371, "4E": 0.0316, "4I": 0.0515, "5E": 0.0755, "5I": 0.0, "6E": 0.0042, "6I": 0.0},
    "4E": {"23E": 0.0077, "23I": 0.0059, "4E": 0.0497, "4I": 0.135, "5E": 0.0067, "5I": 0.0003, "6E": 0.0453, "6I": 0.0},
    "4I": {"23E": 0.0691, "23I": 0.0029, "4E": 0.0794, "4I": 0.1597, "5E": 0.0033, "5I": 0.0, "6E": 0.1057, "6I": 0.0},
    "5E": {"23E": 0.1004, "23I": 0.0622, "4E": 0.0505, "4I": 0.0057, "5E": 0.0831, "5I": 0.3726, "6E": 0.0204, "6I": 0.0},
    "5I": {"23E": 0.0548, "23I": 0.0269, "4E": 0.0257, "4I": 0.0022, "5E": 0.06, "5I": 0.3158, "6E": 0.0086, "6I": 0.0},
    "6E": {"23E": 0.0156, "23I": 0.0066, "4E": 0.0211, "4I": 0.0166, "5E": 0.0572, "5I": 0.0197, "6E": 0.0396, "6I": 0.2252},
    "6I": {"23E": 0.0364, "23I": 0.001, "4E": 0.0034, "4I": 0.0005, "5E": 0.0277, "5I": 0.008, "6E": 0.0658, "6I": 0.1443}}
PD_EXT = {"23E": 1600, "23I": 1500, "4E": 2100, "4I": 1900, "5E": 2000, "5I": 1900, "6E": 2900, "6I": 2100}
PD_RATE = {"23E": 0.971, "23I": 2.868, "4E": 4.746, "4I": 5.396, "5E": 8.142, "5I": 9.078, "6E": 0.991, "6I": 7.523}
PD_MEAN_W = 87.8e-3
PD_G = -4.0
PD_BG_RATE = 8.0
PD_MEAN_DELAY = {"E": 1.5, "I": 0.75}
PD_DELAY_SD = {"E": 0.75, "I": 0.375}
PD_NORM_Q9999 = 3.719016485455709     # scipy.stats.norm.ppf(0.9999)


def pd_full_num_inputs(src, trg):
    n_src, n_trg = PD_NUM[src], PD_NUM[trg]
    p = PD_PROB[trg][src]
    if p == 0.0:
        return 0
    return int(round(math.log(1.0 - p) / math.log(float(n_trg * n_src - 1) / float(n_trg * n_src))) / n_trg)


def pd_mean_weight(src, trg):
    if src.endswith("E"):
        return 2.0 * PD_MEAN_W if (src == "4E" and trg == "23E") else PD_MEAN_W
    return PD_G * PD_MEAN_W


def potjans(neuron_scale=1.0, connectivity_scale=1.0, steps=10000, seed=4321, dt=0.1, pad=4, poisson=False):
    """Scaling rules are those of the reference script (userproject/potjans_microcircuit.py:105-147,
    193-200).  The Poisson background (PoissonExp, currentSourceModels.h:107-129) is replaced by a
    DC source with the same stationary mean, w * tauSyn * rate[1/ms], unless ``poisson`` asks for the
    script's own sources (weight, tauSyn 0.5 ms, rate as in potjans_microcircuit.py:193-200), which draw
    from this build's counter-based generator.  Rows are padded to ``pad`` entries so that row starts
    are 16-byte aligned."""
    pops = [l + p for l in PD_LAYERS for p in ("E", "I")]
    max_delay = {k: PD_MEAN_DELAY[k] + PD_DELAY_SD[k] * PD_NORM_Q9999 for k in ("E", "I")}
    slots = int(round(max(max_delay.values()) / dt))
    net = Net(name="potjans", dt=dt, steps=steps, fuse_psm=True, seed=seed)
    size = {}
    for k, name in enumerate(pops):
        n = int(round(neuron_scale * PD_NUM[name]))
        size[name] = n
        full_in = sum(pd_mean_weight(s, name) * pd_full_num_inputs(s, name) * PD_RATE[s] for s in pops)
        full_in += PD_MEAN_W * PD_EXT[name] * PD_BG_RATE
        ioff = 0.001 * 0.5 * (1.0 - math.sqrt(connectivity_scale)) * full_in
        v0 = (-58.0 + 5.0 * rng.normal(seed, 1 + k, 0, n)).astype(np.float32)
        net.pops.append(Pop(name, "lif", n,
                            dict(C=0.25, TauM=10.0, Vrest=-65.0, Vreset=-65.0, Vthresh=-50.0, Ioffset=ioff, TauRefrac=2.0),
                            {"V": v0, "RefracTime": np.zeros(n, np.float32)}))
        ext_rate = PD_EXT[name] * connectivity_scale * PD_BG_RATE
        ext_w = PD_MEAN_W / math.sqrt(connectivity_scale)
        if poisson:
            net.css.append(CurrentSource(name + "_poisson", "poisson_exp", name, params=dict(weight=ext_w, tauSyn=0.5, rate=ext_rate)))
        else:
            net.css.append(CurrentSource(name + "_dc", "dc", name, amp=ext_w * 0.5 * ext_rate / 1000.0))
    stream = 100
    fmax = float(np.finfo(np.float32).max)
    for trg in pops:
        for src in pops:
            stream += 8
            num_in = pd_full_num_inputs(src, trg) * connectivity_scale
            total = int(round(num_in * float(size[trg])))
            if total <= 0:
                continue
            mean_w = pd_mean_weight(src, trg) / math.sqrt(connectivity_scale)
            sd_w = mean_w * 0.05 if (src == "4E" and trg == "23E") else abs(mean_w * 0.1)
            rl, ind = netgen.fixed_number_total(seed, stream, size[src], size[trg], total, pad=pad)
            stride = ind.shape[1]
            kind = src[-1]
            lo, hi = (0.0, fmax) if kind == "E" else (-fmax, 0.0)
            g = netgen.rows_clipped_normal(seed, stream + 2, rl, stride, mean_w, sd_w, lo, hi)
            d = netgen.rows_clipped_normal_delay(seed, stream + 4, rl, stride, PD_MEAN_DELAY[kind] / dt, PD_DELAY_SD[kind] / dt,
                                                 0.0, max_delay[kind] / dt)
            net.syns.append(Syn(f"{src}_{trg}", src, trg, wum="static_delay", psm="expcurr", tau=0.5,
                                row_stride=stride, row_length=rl, ind=ind, g=g, d=d, max_den_delay=slots))
    return net


# --------------------------------------------------------------------------------------------
# C3: fixed-fanout Izhikevich network with pregenerated noise current
# --------------------------------------------------------------------------------------------
def izhikevich_fanout(n=1_000_000, fanout=1000, steps=1000, seed=777, dt=1.0, noise_steps=None):
    """Regular-spiking Izhikevich neurons, 80/20 excitatory/inhibitory by row, DeltaCurr input.
    ``noise_steps`` rows of U[0,5) noise are generated and cycled (default: one row per step)."""
    n_e = (n * 4) // 5
    net = Net(name="izh", dt=dt, steps=steps, seed=seed)
    v0 = np.full(n, -65.0, np.float32)
    u0 = (np.float32(0.2) * v0).astype(np.float32)
    net.pops.append(Pop("N", "izh", n, dict(a=0.02, b=0.2, c=-65.0, d=8.0), {"V": v0, "U": u0}))
    rl, ind = netgen.fixed_number_post(seed, 10, n, n, fanout)
    g = netgen.rows_uniform(seed, 11, rl, fanout, n_e, 0.5, 0.0, 1.0, -1.0)
    net.syns.append(Syn("NN", "N", "N", wum="static", psm="deltacurr", row_stride=fanout, row_length=rl, ind=ind, g=g))
    rows = steps if noise_steps is None else noise_steps
    noise = netgen.uniform_f32(seed, 12, 0, rows * n, 5.0, 0.0).reshape(rows, n)
    net.css.append(CurrentSource("N_noise", "noise", "N", noise=noise))
    return net


def izhikevich_fanout_snippets(n=1_000_000, fanout=1000, steps=20, seed=777, dt=1.0):
    """The network of :func:`izhikevich_fanout` described by snippets instead of arrays, as a GeNN model would state it:
    excitatory and inhibitory neurons are populations of their own, every population pair a SPARSE projection built by
    FixedNumberPostWithReplacement (the fan-out of 1,000 split 80/20 like the targets) with Uniform weights ([0, 0.5) from
    excitatory, [-1, 0) from inhibitory sources).  Nothing of the matrices exists on the host."""
    n_e = (n * 4) // 5
    net = Net(name="izh_snippets", dt=dt, steps=steps, seed=seed)
    for name, count, stream in (("E", n_e, 12), ("I", n - n_e, 13)):
        v0 = np.full(count, -65.0, np.float32)
        net.pops.append(Pop(name, "izh", count, dict(a=0.02, b=0.2, c=-65.0, d=8.0), {"V": v0, "U": (np.float32(0.2) * v0).astype(np.float32)}))
        net.css.append(CurrentSource(name + "_noise", "noise", name, noise=netgen.uniform_f32(seed, stream, 0, steps * count, 5.0, 0.0).reshape(steps, count)))
    for src, lo, hi in (("E", 0.0, 0.5), ("I", -1.0, 0.0)):
        for trg, share in (("E", (fanout * 4) // 5), ("I", fanout - (fanout * 4) // 5)):
            net.syns.append(Syn(src + trg, src, trg, matrix="sparse_init", wum="static", psm="deltacurr",
                                connect=("FixedNumberPostWithReplacement", {"num": share}), g_init=("Uniform", {"min": lo, "max": hi})))
    return net


# --------------------------------------------------------------------------------------------
# C4: plastic sparse network with trace STDP (pygenn/genn_model.py:1448-1476)
# --------------------------------------------------------------------------------------------
def poisson_spike_source(seed, stream, n, rate_hz, steps, dt, rates=None):
    """Pregenerated Poisson spike times (ms, on the dt grid) in SpikeSourceArray layout
    (startSpike/endSpike/spikeTimes, include/genn/genn/neuronModels.h:274-286)."""
    p = (np.full(n, rate_hz) if rates is None else np.asarray(rates)) * dt / 1000.0
    u = netgen.uniform_f32(seed, stream, 0, n * steps).reshape(n, steps)
    fire = u < p[:, None].astype(np.float32)
    counts = fire.sum(axis=1)
    end = np.cumsum(counts).astype(np.uint32)
    start = (end - counts).astype(np.uint32)
    _, step = np.nonzero(fire)
    times = (step.astype(np.float64) * dt).astype(np.float32)
    return start, end, times


def plastic_stdp(n=100_000, n_src=1000, steps=10000, seed=99, dt=1.0, fan=500, src_fan=100, src_w=2.0,
                 ioffset=0.45, w_ei=0.25, w_ie=-1.0, w_ii=-1.0, rule="stdp_trace"):
    """80 % excitatory neurons with plastic E->E (fanout ~``fan``, g0 ~ U[0,0.5], clipped to [0,1]); the
    static E->I, I->E, I->I projections close a balanced loop; Poisson sources drive E.  ``rule``: "stdp_trace"
    (pygenn/genn_model.py:1448-1476) or "stdp_additive" (the built-in nearest-neighbour rule, weightUpdateModels.h:345-367)."""
    n_e = (n * 4) // 5
    n_i = n - n_e
    net = Net(name="stdp", dt=dt, steps=steps, seed=seed)
    lif = dict(C=1.0, TauM=20.0, Vrest=-60.0, Vreset=-60.0, Vthresh=-50.0, Ioffset=ioffset, TauRefrac=5.0)
    for k, (name, num) in enumerate((("E", n_e), ("I", n_i))):
        v0 = (-60.0 + 10.0 * rng.uniform(seed, 1 + k, 0, num)).astype(np.float32)
        net.pops.append(Pop(name, "lif", num, dict(lif), {"V": v0, "RefracTime": np.zeros(num, np.float32)}))
    start, end, times = poisson_spike_source(seed, 5, n_src, 10.0, steps, dt)
    net.pops.append(Pop("P", "ssa", n_src, {}, {"startSpike": start, "endSpike": end}, spike_times=times))
    p_conn = min(1.0, fan / n_e)
    rl, ind = netgen.fixed_probability(seed, 20, n_e, n_e, p_conn)
    g = netgen.rows_uniform(seed, 21, rl, ind.shape[1], n_e, 0.5, 0.0, 0.5, 0.0)
    net.syns.append(Syn("EE", "E", "E", wum=rule,
                        wum_params=dict(tauPlus=20.0, tauMinus=20.0, aPlus=0.01, aMinus=0.012, wMin=0.0, wMax=1.0),
                        psm="expcurr", tau=5.0, row_stride=ind.shape[1], row_length=rl, ind=ind, g=g))
    for name, src, trg, ns, nt, w, tau, st in (("EI", "E", "I", n_e, n_i, w_ei, 5.0, 22), ("IE", "I", "E", n_i, n_e, w_ie, 10.0, 23),
                                               ("II", "I", "I", n_i, n_i, w_ii, 10.0, 24)):
        rl, ind = netgen.fixed_probability(seed, st, ns, nt, p_conn)
        net.syns.append(Syn(name, src, trg, wum="static", psm="expcurr", tau=tau, row_stride=ind.shape[1],
                            row_length=rl, ind=ind, g=_const_rows(rl, ind.shape[1], w)))
    rl, ind = netgen.fixed_number_post(seed, 25, n_src, n_e, min(src_fan, n_e))
    net.syns.append(Syn("PE", "P", "E", wum="static", psm="expcurr", tau=5.0, row_stride=ind.shape[1],
                        row_length=rl, ind=ind, g=np.full(ind.shape, np.float32(src_w), np.float32)))
    return net


# --------------------------------------------------------------------------------------------
# C5: convolutional spiking layer through TOEPLITZ connectivity
# --------------------------------------------------------------------------------------------
def conv_toeplitz(h=64, w=64, ic=16, oc=32, k=3, steps=500, seed=5, dt=1.0, batch_index=0, max_rate=50.0, w_sd=0.1,
                  ioffset=0.0):
    """Rate-coded Poisson sources (rates U[0,max_rate) Hz, one spike train per batch index) into a LIF
    layer through Conv2D k x k, stride 1, same padding; kernel weights N(0, w_sd)."""
    n_in, n_out = h * w * ic, h * w * oc
    net = Net(name="conv", dt=dt, steps=steps, seed=seed)
    rates = max_rate * rng.uniform(seed, 1, 0, n_in)
    start, end, times = poisson_spike_source(seed, 100 + batch_index, n_in, 0.0, steps, dt, rates=rates)
    net.pops.append(Pop("In", "ssa", n_in, {}, {"startSpike": start, "endSpike": end}, spike_times=times))
    lif = dict(C=1.0, TauM=20.0, Vrest=-60.0, Vreset=-60.0, Vthresh=-50.0, Ioffset=ioffset, TauRefrac=5.0)
    net.pops.append(Pop("Out", "lif", n_out, lif, {"V": np.full(n_out, -60.0, np.float32), "RefracTime": np.zeros(n_out, np.float32)}))
    kern = (w_sd * rng.normal(seed, 2, 0, k * k * ic * oc)).astype(np.float32).reshape(k, k, ic, oc)
    net.syns.append(Syn("Conv", "In", "Out", matrix="conv2d", wum="static", psm="expcurr", tau=5.0, g=kern,
                        conv=dict(conv_kh=k, conv_kw=k, conv_ih=h, conv_iw=w, conv_ic=ic, conv_oh=h, conv_ow=w, conv_oc=oc)))
    return net


def dense_bitmask(n_a=300, n_b=77, steps=200, seed=9, dt=1.0, fuse=False):
    """Recurrent LIF network over the remaining matrix types: DENSE with individual weights (A -> B), BITMASK with a
    constant weight (B -> A), DENSE with a constant weight (A -> A) and SPARSE with a constant weight (B -> B).  Sizes
    that are no multiple of a wavefront or of a 32-bit connectivity word."""
    lif = dict(C=1.0, TauM=20.0, Vrest=-60.0, Vreset=-60.0, Vthresh=-50.0, Ioffset=0.6, TauRefrac=2.0)
    net = Net(name="dense_bitmask", dt=dt, steps=steps, fuse_psm=fuse, seed=seed)
    net.pops.append(Pop("A", "lif", n_a, dict(lif), {"V": (-60.0 + 9.0 * rng.uniform(seed, 1, 0, n_a)).astype(np.float32),
                                                     "RefracTime": np.zeros(n_a, np.float32)}))
    net.pops.append(Pop("B", "lif", n_b, dict(lif, Ioffset=0.45), {"V": (-60.0 + 9.0 * rng.uniform(seed, 2, 0, n_b)).astype(np.float32),
                                                                   "RefracTime": np.zeros(n_b, np.float32)}))
    g_ab = (0.02 * rng.normal(seed, 3, 0, n_a * n_b)).astype(np.float32).reshape(n_a, n_b)
    net.syns.append(Syn("AB_dense", "A", "B", matrix="dense", wum="static", psm="expcurr", tau=5.0, g=g_ab))
    stride = (n_a + 31) // 32 * 32
    bits = np.zeros((n_b, stride), np.uint8)
    bits[:, :n_a] = rng.uniform(seed, 4, 0, n_b * n_a).reshape(n_b, n_a) < 0.2
    gp = np.packbits(bits.reshape(-1), bitorder="big").view(">u4").astype(np.uint32)       # most significant bit of a word first
    net.syns.append(Syn("BA_bitmask", "B", "A", matrix="bitmask", wum="static_const", wum_params={"g": -0.08}, psm="expcurr", tau=5.0,
                        gp=gp, row_stride=stride))
    net.syns.append(Syn("AA_dense_const", "A", "A", matrix="dense", wum="static_const", wum_params={"g": 0.0005}, psm="expcurr", tau=5.0))
    ind = np.sort(rng.randint(seed, 5, 0, n_b * 20, n_b).reshape(n_b, 20), axis=1).astype(np.uint32)
    net.syns.append(Syn("BB_sparse_const", "B", "B", wum="static_const", wum_params={"g": 0.03}, psm="expcurr", tau=5.0,
                        row_stride=20, row_length=np.full(n_b, 20, np.uint32), ind=ind))
    return net


def graded(n_a=300, n_b=130, n_c=64, steps=200, seed=13, dt=0.5):
    """Graded (spike-like event) transmission next to ordinary spikes: two LIF populations and an Izhikevich one, three
    StaticGraded projections with different thresholds and slopes (two of them leave population A, so it keeps two event
    queues) and one spiking inhibitory projection back."""
    lif = dict(C=1.0, TauM=20.0, Vrest=-60.0, Vreset=-60.0, Vthresh=-50.0, Ioffset=0.6, TauRefrac=2.0)
    net = Net(name="graded", dt=dt, steps=steps, seed=seed)
    net.pops.append(Pop("A", "lif", n_a, dict(lif), {"V": (-60.0 + 9.0 * rng.uniform(seed, 1, 0, n_a)).astype(np.float32),
                                                     "RefracTime": np.zeros(n_a, np.float32)}))
    net.pops.append(Pop("B", "lif", n_b, dict(lif, Ioffset=0.35), {"V": (-60.0 + 5.0 * rng.uniform(seed, 2, 0, n_b)).astype(np.float32),
                                                                   "RefracTime": np.zeros(n_b, np.float32)}))
    net.pops.append(Pop("C", "izh", n_c, dict(a=0.02, b=0.2, c=-65.0, d=8.0),
                        {"V": (-65.0 + 10.0 * rng.uniform(seed, 3, 0, n_c)).astype(np.float32), "U": np.full(n_c, -13.0, np.float32)}))
    net.css.append(CurrentSource("C_dc", "dc", "C", amp=6.0))

    def sparse(name, src, trg, n_src, n_trg, stride, stream, lo, hi, **kw):
        ind = np.sort(rng.randint(seed, stream, 0, n_src * stride, n_trg).reshape(n_src, stride), axis=1).astype(np.uint32)
        row_length = (stride - rng.randint(seed, stream + 1, 0, n_src, 4)).astype(np.uint32)          # ragged rows
        g = (lo + (hi - lo) * rng.uniform(seed, stream + 2, 0, n_src * stride)).astype(np.float32).reshape(n_src, stride)
        return Syn(name, src, trg, psm="expcurr", row_stride=stride, row_length=row_length, ind=ind, g=g, **kw)

    net.syns.append(sparse("AB_graded", "A", "B", n_a, n_b, 24, 10, 0.0, 0.04, wum="static_graded",
                           wum_params={"Epre": -54.3, "Vslope": 7.3}, tau=5.0))
    net.syns.append(sparse("AA_graded", "A", "A", n_a, n_a, 16, 20, -0.01, 0.03, wum="static_graded",
                           wum_params={"Epre": -52.0, "Vslope": 4.1}, tau=8.0))
    net.syns.append(sparse("CB_graded", "C", "B", n_c, n_b, 40, 30, 0.0, 0.02, wum="static_graded",
                           wum_params={"Epre": -40.0, "Vslope": 20.0}, tau=5.0))
    net.syns.append(sparse("BA_spikes", "B", "A", n_b, n_a, 30, 40, -0.6, -0.2, wum="static", tau=10.0))
    return net


def reverse(n_a=260, n_b=90, steps=200, seed=21, dt=1.0):
    """Presynaptic ("reverse") output: population A spikes, and every synapse of its projection to B adds its weight to
    the spiking neuron's own input (`addToPre(g)`), here a self-inhibition that grows with the neuron's out-degree; B
    projects back the ordinary way, and has a reverse projection of its own onto a sparser matrix."""
    lif = dict(C=1.0, TauM=20.0, Vrest=-60.0, Vreset=-60.0, Vthresh=-50.0, Ioffset=0.7, TauRefrac=2.0)
    net = Net(name="reverse", dt=dt, steps=steps, seed=seed)
    net.pops.append(Pop("A", "lif", n_a, dict(lif), {"V": (-60.0 + 9.5 * rng.uniform(seed, 1, 0, n_a)).astype(np.float32),
                                                     "RefracTime": np.zeros(n_a, np.float32)}))
    net.pops.append(Pop("B", "lif", n_b, dict(lif, Ioffset=0.58), {"V": (-60.0 + 9.5 * rng.uniform(seed, 2, 0, n_b)).astype(np.float32),
                                                                   "RefracTime": np.zeros(n_b, np.float32)}))

    def sparse(name, src, trg, n_src, n_trg, stride, stream, lo, hi, wum):
        ind = np.sort(rng.randint(seed, stream, 0, n_src * stride, n_trg).reshape(n_src, stride), axis=1).astype(np.uint32)
        row_length = (stride - rng.randint(seed, stream + 1, 0, n_src, stride // 2)).astype(np.uint32)    # ragged: half to full rows
        g = (lo + (hi - lo) * rng.uniform(seed, stream + 2, 0, n_src * stride)).astype(np.float32).reshape(n_src, stride)
        return Syn(name, src, trg, psm="expcurr", tau=5.0, row_stride=stride, row_length=row_length, ind=ind, g=g, wum=wum)

    net.syns.append(sparse("AB_reverse", "A", "B", n_a, n_b, 36, 10, -0.8, 0.1, "static_reverse"))
    net.syns.append(sparse("AB_forward", "A", "B", n_a, n_b, 12, 20, 0.0, 0.08, "static"))
    net.syns.append(sparse("BA_forward", "B", "A", n_b, n_a, 20, 30, -0.2, 0.1, "static"))
    net.syns.append(sparse("BA_reverse", "B", "A", n_b, n_a, 7, 40, -1.5, 0.0, "static_reverse"))
    return net


def procedural(n_e=1600, n_i=400, steps=200, seed=31, dt=1.0, order_free=False):
    """Recurrent LIF network whose four projections are PROCEDURAL: FixedProbability[NoAutapse] and
    FixedNumberPostWithReplacement connectivity, constant, Uniform and Normal weights.  Nothing is stored: the matrices are a
    function of the seed.  ``order_free``: one dyadic weight per projection into DeltaCurr inputs, so that every sum is exact
    in any order and two executors that regenerate the same matrices stay identical for ever."""
    lif = dict(C=1.0, TauM=20.0, Vrest=-60.0, Vreset=-60.0, Vthresh=-50.0, Ioffset=0.56, TauRefrac=2.0)
    net = Net(name="procedural", dt=dt, steps=steps, seed=seed)
    net.pops.append(Pop("E", "lif", n_e, dict(lif), {"V": (-60.0 + 10.0 * rng.uniform(seed, 1, 0, n_e)).astype(np.float32), "RefracTime": np.zeros(n_e, np.float32)}))
    net.pops.append(Pop("I", "lif", n_i, dict(lif), {"V": (-60.0 + 10.0 * rng.uniform(seed, 2, 0, n_i)).astype(np.float32), "RefracTime": np.zeros(n_i, np.float32)}))
    net.syns.append(Syn("EE", "E", "E", matrix="procedural", wum="static", psm="expcurr", tau=5.0,
                        connect=("FixedProbabilityNoAutapse", {"prob": 0.05}), g_init=("Uniform", {"min": 0.0, "max": 0.1})))
    net.syns.append(Syn("EI", "E", "I", matrix="procedural", wum="static_const", wum_params={"g": 0.05}, psm="expcurr", tau=5.0,
                        connect=("FixedNumberPostWithReplacement", {"num": 20})))
    net.syns.append(Syn("IE", "I", "E", matrix="procedural", wum="static", psm="expcurr", tau=10.0,
                        connect=("FixedProbability", {"prob": 0.05}), g_init=("Normal", {"mean": -0.3, "sd": 0.05})))
    net.syns.append(Syn("II", "I", "I", matrix="procedural", wum="static", psm="expcurr", tau=10.0,
                        connect=("FixedNumberPostWithReplacement", {"num": 300}), g_init=("Constant", {"constant": -0.3})))
    if order_free:
        for s, w in zip(net.syns, (0.015625, 0.03125, -0.0625, -0.0625)):
            s.psm = "deltacurr"
            if s.wum == "static_const":
                s.wum_params = {"g": w}
            else:
                s.g_init = ("Constant", {"constant": w})
    return net


def snippet_initialised(n_e=1600, n_i=400, steps=200, seed=31, dt=1.0):
    """The network of :func:`procedural` with its four projections stored: SPARSE matrices whose connectivity and weights are
    built by the same snippets at initialisation time."""
    net = procedural(n_e=n_e, n_i=n_i, steps=steps, seed=seed, dt=dt)
    net.name = "snippet_initialised"
    for s in net.syns:
        s.matrix = "sparse_init"
    return net


def snippet_initialised_layers(steps=200, seed=37, dt=1.0):
    """A small feed-forward network whose stored SPARSE matrices are built by the remaining built-in snippets: Poisson
    sources on an 8 x 8 x 2 grid drive an 8 x 8 x 4 layer through Conv2D connectivity with kernel-initialised weights
    (3 x 3, stride 1, padding 1), the layer drives a read-out population through FixedNumberPreWithReplacement with Uniform
    weights, and the read-out inhibits the layer through FixedNumberPreWithReplacement with one weight."""
    net = Net(name="snippet_initialised_layers", dt=dt, steps=steps, seed=seed)
    shape = dict(conv_kh=3, conv_kw=3, conv_sh=1, conv_sw=1, conv_padh=1, conv_padw=1, conv_ih=8, conv_iw=8, conv_ic=2, conv_oh=8, conv_ow=8, conv_oc=4)
    n_in, n_mid, n_out = 8 * 8 * 2, 8 * 8 * 4, 200
    start, end, times = poisson_spike_source(seed, 1, n_in, 80.0, steps, dt)
    net.pops.append(Pop("In", "ssa", n_in, {}, {"startSpike": start, "endSpike": end}, spike_times=times))
    lif = dict(C=1.0, TauM=20.0, Vrest=-60.0, Vreset=-60.0, Vthresh=-50.0, Ioffset=0.35, TauRefrac=2.0)
    net.pops.append(Pop("Mid", "lif", n_mid, dict(lif), {"V": (-60.0 + 9.0 * rng.uniform(seed, 2, 0, n_mid)).astype(np.float32), "RefracTime": np.zeros(n_mid, np.float32)}))
    net.pops.append(Pop("Out", "lif", n_out, dict(lif, Ioffset=0.2), {"V": (-60.0 + 9.0 * rng.uniform(seed, 3, 0, n_out)).astype(np.float32), "RefracTime": np.zeros(n_out, np.float32)}))
    kernel = (0.05 + 0.25 * rng.uniform(seed, 4, 0, 3 * 3 * 2 * 4)).astype(np.float32).reshape(3, 3, 2, 4)
    net.syns.append(Syn("InMid", "In", "Mid", matrix="sparse_init", wum="static", psm="expcurr", tau=5.0,
                        connect=("Conv2D", shape), g_init=("Kernel", {"kernel": kernel})))
    net.syns.append(Syn("MidOut", "Mid", "Out", matrix="sparse_init", wum="static", psm="expcurr", tau=5.0,
                        connect=("FixedNumberPreWithReplacement", {"num": 30}), g_init=("Uniform", {"min": 0.0, "max": 0.08})))
    net.syns.append(Syn("OutMid", "Out", "Mid", matrix="sparse_init", wum="static_const", wum_params={"g": -0.05}, psm="expcurr", tau=10.0,
                        connect=("FixedNumberPreWithReplacement", {"num": 10})))
    return net


def dense_layer(n_in=8192, n_out=8192, rate_hz=50.0, steps=1000, seed=17, dt=1.0, w_sd=0.02):
    """A fully connected spiking layer: Poisson sources (rate_hz per source) into LIF neurons through a DENSE matrix
    with individual weights ~ N(0, w_sd); the shape of the dense layers of rate-coded classifiers."""
    net = Net(name="dense_layer", dt=dt, steps=steps, seed=seed)
    start, end, times = poisson_spike_source(seed, 1, n_in, rate_hz, steps, dt)
    net.pops.append(Pop("In", "ssa", n_in, {}, {"startSpike": start, "endSpike": end}, spike_times=times))
    lif = dict(C=1.0, TauM=20.0, Vrest=-60.0, Vreset=-60.0, Vthresh=-50.0, Ioffset=0.3, TauRefrac=2.0)
    net.pops.append(Pop("Out", "lif", n_out, lif, {"V": np.full(n_out, -60.0, np.float32), "RefracTime": np.zeros(n_out, np.float32)}))
    g = netgen.normal_f32(seed, 2, 0, n_in * n_out, 0.0, w_sd).reshape(n_in, n_out)
    net.syns.append(Syn("InOut", "In", "Out", matrix="dense", wum="static", psm="expcurr", tau=5.0, g=g))
    return net


def poisson_input(n_in=1500, n_out=400, rate=20.0, steps=1000, seed=53, dt=1.0):
    """A population of the built-in Poisson neuron (neuronModels.h:307-325: a countdown to the next spike, refilled with
    isi * gennrand_exponential()) driving LIF neurons through a static SPARSE projection.  The model draws random numbers
    while it runs, from whatever generator its backend has — no two backends of the reference produce the same spikes —
    so what can be compared is statistics.  On the MI355X backend the neuron's code reaches the generated kernels."""
    net = Net(name="poisson_input", dt=dt, steps=steps, seed=seed)
    net.pops.append(Pop("In", "poisson", n_in, {"rate": rate}, {"timeStepToSpike": np.zeros(n_in, np.float32)}))
    lif = dict(C=1.0, TauM=20.0, Vrest=-60.0, Vreset=-60.0, Vthresh=-50.0, Ioffset=0.0, TauRefrac=2.0)
    net.pops.append(Pop("Out", "lif", n_out, lif, {"V": (-60.0 + 9.0 * rng.uniform(seed, 1, 0, n_out)).astype(np.float32),
                                                      "RefracTime": np.zeros(n_out, np.float32)}))
    stride = 40
    ind = np.sort(rng.randint(seed, 2, 0, n_in * stride, n_out).reshape(n_in, stride), axis=1).astype(np.uint32)
    g = (0.02 + 0.06 * rng.uniform(seed, 3, 0, n_in * stride)).astype(np.float32).reshape(n_in, stride)
    net.syns.append(Syn("InOut", "In", "Out", psm="expcurr", tau=5.0, row_stride=stride, row_length=np.full(n_in, stride, np.uint32),
                        ind=ind, g=g, wum="static"))
    return net


def synapse_dynamics(n_a=240, n_b=160, steps=300, seed=67, dt=1.0):
    """Weight-update code that runs for every synapse every step ("leaky_graded", a model of the test driver: each synapse keeps
    a decaying trace of how far its source's membrane potential is above a midpoint and delivers g times the trace, spike or
    no spike) between two LIF populations, beside an ordinary static inhibitory projection.  Exists only as code strings of
    the driver's model class, so on the MI355X backend it runs through generated kernels."""
    lif = dict(C=1.0, TauM=20.0, Vrest=-60.0, Vreset=-60.0, Vthresh=-50.0, Ioffset=0.55, TauRefrac=2.0)
    net = Net(name="synapse_dynamics", dt=dt, steps=steps, seed=seed)
    net.pops.append(Pop("A", "lif", n_a, lif, {"V": (-60.0 + 9.5 * rng.uniform(seed, 1, 0, n_a)).astype(np.float32), "RefracTime": np.zeros(n_a, np.float32)}))
    net.pops.append(Pop("B", "lif", n_b, dict(lif, Ioffset=0.2), {"V": (-60.0 + 9.5 * rng.uniform(seed, 2, 0, n_b)).astype(np.float32),
                                                                    "RefracTime": np.zeros(n_b, np.float32)}))

    def sparse(name, src, trg, n_src, n_trg, stride, stream, lo, hi, wum, tau, params=None):
        ind = np.sort(rng.randint(seed, stream, 0, n_src * stride, n_trg).reshape(n_src, stride), axis=1).astype(np.uint32)
        row_length = (stride - rng.randint(seed, stream + 1, 0, n_src, stride // 3)).astype(np.uint32)
        g = (lo + (hi - lo) * rng.uniform(seed, stream + 2, 0, n_src * stride)).astype(np.float32).reshape(n_src, stride)
        return Syn(name, src, trg, psm="expcurr", tau=tau, row_stride=stride, row_length=row_length, ind=ind, g=g, wum=wum, wum_params=params or {})

    net.syns.append(sparse("AB_graded", "A", "B", n_a, n_b, 24, 10, 0.0, 0.004, "leaky_graded", 5.0, {"Vmid": -56.0, "decay": 0.8}))
    net.syns.append(sparse("BA_inhibit", "B", "A", n_b, n_a, 20, 20, -0.4, -0.1, "static", 10.0))
    return net


def stochastic_synapses(n_a=400, n_b=300, steps=600, seed=71, dt=1.0, twin=False):
    """Synapses that transmit with a probability ("stochastic", a model of the test driver: `if(gennrand_uniform() < pRelease)
    addToPost(g)`): a driven LIF population A onto B, whose threshold is out of reach so that its membrane potential is a
    linear functional of its input, through synapses that release 40 % of the time, and onto spiking C through synapses that
    always release.  `twin`: the same network with static synapses — weights times 0.4 onto B (the expectation of the
    stochastic input), unchanged onto C (the same input exactly)."""
    lif = dict(C=1.0, TauM=20.0, Vrest=-60.0, Vreset=-60.0, Vthresh=-50.0, Ioffset=0.0, TauRefrac=2.0)
    net = Net(name="stochastic_twin" if twin else "stochastic", dt=dt, steps=steps, seed=seed)
    net.pops.append(Pop("A", "lif", n_a, dict(lif, Ioffset=0.75), {"V": (-60.0 + 9.5 * rng.uniform(seed, 1, 0, n_a)).astype(np.float32),
                                                                   "RefracTime": np.zeros(n_a, np.float32)}))
    net.pops.append(Pop("B", "lif", n_b, dict(lif, Vthresh=1.0e9), {"V": np.full(n_b, -60.0, np.float32), "RefracTime": np.zeros(n_b, np.float32)}))
    net.pops.append(Pop("C", "lif", n_b, lif, {"V": np.full(n_b, -60.0, np.float32), "RefracTime": np.zeros(n_b, np.float32)}))
    stride = 60
    ind = np.sort(rng.randint(seed, 2, 0, n_a * stride, n_b).reshape(n_a, stride), axis=1).astype(np.uint32)
    g = (0.05 + 0.1 * rng.uniform(seed, 3, 0, n_a * stride)).astype(np.float32).reshape(n_a, stride)
    common = dict(psm="expcurr", tau=5.0, row_stride=stride, row_length=np.full(n_a, stride, np.uint32), ind=ind)
    if twin:
        net.syns.append(Syn("AB", "A", "B", g=(g * np.float32(0.4)).astype(np.float32), wum="static", **common))
        net.syns.append(Syn("AC", "A", "C", g=g, wum="static", **common))
    else:
        net.syns.append(Syn("AB", "A", "B", g=g, wum="stochastic", wum_params={"pRelease": 0.4}, **common))
        net.syns.append(Syn("AC", "A", "C", g=g, wum="stochastic", wum_params={"pRelease": 1.0}, **common))
    return net


def custom_models(n_a=300, n_b=200, steps=300, seed=41, dt=1.0, timing="timing_copy"):
    """A network of models that are NOT built into GeNN or into the device library — what a user writes with the model
    API: LIF neurons with a spike-triggered adaptation variable ("lifa": the built-in LIF plus A, which decays every step,
    is subtracted from the input and grows by dA at each spike), and a weight update model with a presynaptic and a
    postsynaptic variable after tests/features/test_wu_vars.py ("timing_copy": each neuron's variable holds the time of
    its last spike; a presynaptic spike delivers g and copies the target's variable into the row's synapses, a
    postsynaptic spike copies the source's variable into its column).  Their code exists only as strings of the test
    driver's model classes, so on the MI355X backend this network runs through generated kernels."""
    lifa = dict(C=1.0, TauM=20.0, Vrest=-60.0, Vreset=-60.0, Vthresh=-50.0, Ioffset=0.9, TauRefrac=2.0, TauA=50.0, dA=0.12)
    net = Net(name="custom", dt=dt, steps=steps, seed=seed)
    for k, (name, n, ioff) in enumerate((("A", n_a, 0.9), ("B", n_b, 0.45))):
        net.pops.append(Pop(name, "lifa", n, dict(lifa, Ioffset=ioff),
                            {"V": (-60.0 + 9.5 * rng.uniform(seed, 1 + k, 0, n)).astype(np.float32), "RefracTime": np.zeros(n, np.float32),
                             "A": (0.1 * rng.uniform(seed, 5 + k, 0, n)).astype(np.float32)}))

    def sparse(name, src, trg, n_src, n_trg, stride, stream, lo, hi, wum, tau):
        ind = np.sort(rng.randint(seed, stream, 0, n_src * stride, n_trg).reshape(n_src, stride), axis=1).astype(np.uint32)
        row_length = (stride - rng.randint(seed, stream + 1, 0, n_src, stride // 3)).astype(np.uint32)
        g = (lo + (hi - lo) * rng.uniform(seed, stream + 2, 0, n_src * stride)).astype(np.float32).reshape(n_src, stride)
        return Syn(name, src, trg, psm="expcurr", tau=tau, row_stride=stride, row_length=row_length, ind=ind, g=g, wum=wum)

    net.syns.append(sparse("AB_timing", "A", "B", n_a, n_b, 30, 10, 0.0, 0.12, timing, 5.0))
    net.syns.append(sparse("BA_inhibit", "B", "A", n_b, n_a, 24, 20, -0.5, -0.1, "static", 10.0))
    net.syns.append(sparse("AA_timing", "A", "A", n_a, n_a, 70, 30, 0.0, 0.02, timing, 5.0))
    return net


def custom_updates(n_a=200, n_b=90, steps=200, seed=57, dt=1.0):
    """A network with custom updates — functions of the model that the user calls between steps (Runtime::customUpdate),
    after tests/features/test_custom_update.py: every 20 steps population B's membrane potentials are pulled towards rest
    and population A's are summed and maximised over the population; every 30 steps the plastic A -> B weights and the
    dense A -> B weights decay (each update accumulating into a variable of its own) and the decayed dense matrix is
    transposed into the dense B -> A projection's weights; every 50 steps the plastic weights are reduced over batches."""
    lif = dict(C=1.0, TauM=20.0, Vrest=-60.0, Vreset=-60.0, Vthresh=-50.0, Ioffset=0.7, TauRefrac=2.0)
    net = Net(name="custom_update", dt=dt, steps=steps, seed=seed)
    net.pops.append(Pop("A", "lif", n_a, dict(lif), {"V": (-60.0 + 9.5 * rng.uniform(seed, 1, 0, n_a)).astype(np.float32),
                                                     "RefracTime": np.zeros(n_a, np.float32)}))
    net.pops.append(Pop("B", "lif", n_b, dict(lif, Ioffset=0.4), {"V": (-60.0 + 9.5 * rng.uniform(seed, 2, 0, n_b)).astype(np.float32),
                                                                  "RefracTime": np.zeros(n_b, np.float32)}))
    stride = 24
    ind = np.sort(rng.randint(seed, 10, 0, n_a * stride, n_b).reshape(n_a, stride), axis=1).astype(np.uint32)
    # (a target at most once per row: the plastic rule and the decay both own their synapse)
    row_length = np.zeros(n_a, np.uint32)
    for i in range(n_a):
        row = np.unique(ind[i])
        row_length[i] = len(row)
        ind[i, :len(row)] = row
        ind[i, len(row):] = 0
    g = (0.05 + 0.25 * rng.uniform(seed, 11, 0, n_a * stride)).astype(np.float32).reshape(n_a, stride)
    net.syns.append(Syn("AB_plastic", "A", "B", wum="stdp_trace",
                        wum_params=dict(tauPlus=20.0, tauMinus=20.0, aPlus=0.01, aMinus=0.012, wMin=0.0, wMax=1.0),
                        psm="expcurr", tau=5.0, row_stride=stride, row_length=row_length, ind=ind, g=g))
    g_ab = (0.004 * rng.uniform(seed, 12, 0, n_a * n_b)).astype(np.float32).reshape(n_a, n_b)
    net.syns.append(Syn("AB_dense", "A", "B", matrix="dense", wum="static", psm="expcurr", tau=5.0, g=g_ab))
    # (its weights are overwritten by the transpose: until the first call it carries these)
    g_ba = (-0.002 * rng.uniform(seed, 13, 0, n_b * n_a)).astype(np.float32).reshape(n_b, n_a)
    net.syns.append(Syn("BA_dense", "B", "A", matrix="dense", wum="static", psm="expcurr", tau=10.0, g=g_ba))
    net.customs.append(Custom("BDecay", "Homeostasis", "decay", "B", params=dict(rest=-60.0, factor=0.5)))
    net.customs.append(Custom("ASum", "Homeostasis", "neuron_reduce", "A"))
    net.customs.append(Custom("PlasticDecay", "Decay", "wu_decay", "AB_plastic", params=dict(factor=0.9)))
    net.customs.append(Custom("DenseDecay", "Decay", "wu_decay", "AB_dense", params=dict(factor=0.75)))
    net.customs.append(Custom("Feedback", "Decay", "transpose", "AB_dense", "BA_dense"))
    net.customs.append(Custom("PlasticReduce", "Reduce", "batch_reduce", "AB_plastic"))
    net.custom_calls += [("Homeostasis", 20), ("Decay", 30), ("Reduce", 50)]
    return net


def rewiring(steps=200):
    """The plastic network of :func:`custom_updates` with custom CONNECTIVITY updates (structural plasticity): every 40
    steps synapses of the plastic projection whose weight has fallen below a threshold are removed (the row's last synapse
    moves into the gap, with every variable that lives on the synapses), every 25 steps each row that has room sprouts a
    synapse onto a target that moves on from call to call; in between the weights keep learning and decaying.  The
    projection learns from postsynaptic spikes, so its column view is rebuilt after every change."""
    net = custom_updates(steps=steps)
    net.name = "rewiring"
    net.customs = [c for c in net.customs if c.name == "PlasticDecay"]
    net.syn("AB_plastic").col_stride = 128          # room for the columns to grow
    net.customs.append(Custom("Prune", "Prune", "prune", "AB_plastic", params=dict(threshold=0.12)))
    net.customs.append(Custom("Sprout", "Sprout", "sprout", "AB_plastic", params=dict(weight=0.2)))
    net.custom_calls = [("Decay", 30), ("Prune", 40), ("Sprout", 25)]
    return net


def post_events(n_a=300, n_b=130, steps=200, seed=23, dt=1.0):
    """Postsynaptic spike-like events: a projection whose synapses, while their TARGET's membrane potential is above a midpoint,
    count the step and send a fraction of their weight back to their source (a model of the test driver after
    tests/features/test_event_propagation.py), beside a plain inhibitory projection back."""
    lif = dict(C=1.0, TauM=20.0, Vrest=-60.0, Vreset=-60.0, Vthresh=-50.0, Ioffset=0.55, TauRefrac=2.0)
    net = Net(name="post_events", dt=dt, steps=steps, seed=seed)
    net.pops.append(Pop("A", "lif", n_a, dict(lif), {"V": (-60.0 + 9.5 * rng.uniform(seed, 1, 0, n_a)).astype(np.float32),
                                                     "RefracTime": np.zeros(n_a, np.float32)}))
    net.pops.append(Pop("B", "lif", n_b, dict(lif, Ioffset=0.45), {"V": (-60.0 + 9.5 * rng.uniform(seed, 2, 0, n_b)).astype(np.float32),
                                                                   "RefracTime": np.zeros(n_b, np.float32)}))

    def sparse(name, src, trg, n_src, n_trg, stride, stream, lo, hi, **kw):
        ind = np.sort(rng.randint(seed, stream, 0, n_src * stride, n_trg).reshape(n_src, stride), axis=1).astype(np.uint32)
        row_length = (stride - rng.randint(seed, stream + 1, 0, n_src, stride // 3)).astype(np.uint32)
        g = (lo + (hi - lo) * rng.uniform(seed, stream + 2, 0, n_src * stride)).astype(np.float32).reshape(n_src, stride)
        return Syn(name, src, trg, psm="expcurr", tau=5.0, row_stride=stride, row_length=row_length, ind=ind, g=g, **kw)

    net.syns.append(sparse("AB_feedback", "A", "B", n_a, n_b, 20, 10, 0.0, 0.1, wum="post_event", wum_params=dict(Vmid=-53.0, back=0.002)))
    net.syns.append(sparse("BA_inhibit", "B", "A", n_b, n_a, 30, 20, -0.3, -0.05, wum="static"))
    return net
