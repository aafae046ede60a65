"""Plain-data description of a spiking network: populations, current sources, projections.

This is the one description every executor consumes: the MI355X engine (through the C-ABI),
the CPU oracle under ``oracle/`` (tests and the bench's CPU baseline only) and, in the
builder container, the reference's own SingleThreadedCPU backend via ``oracle/ref_driver.cc``
(which reads the directory written by :func:`write_netspec`).  All arrays use the reference's
ragged SPARSE layout (``rowLength[numPre]``, ``ind/g/d[numPre*rowStride]`` with identical
padding; src/genn/genn/runtime/runtime.cc:360-402).
"""
from dataclasses import dataclass, field
from typing import Dict, List, Optional
import hashlib
import os

import numpy as np

NEURON_MODELS = ("lif", "izh", "ssa")
LIF_PARAMS = ("C", "TauM", "Vrest", "Vreset", "Vthresh", "Ioffset", "TauRefrac")
IZH_PARAMS = ("a", "b", "c", "d")
STDP_PARAMS = ("tauPlus", "tauMinus", "aPlus", "aMinus", "wMin", "wMax")
CONV_PARAMS = ("conv_kh", "conv_kw", "conv_ih", "conv_iw", "conv_ic", "conv_oh", "conv_ow", "conv_oc")
# Conv2D as SPARSE connectivity (initSparseConnectivitySnippet.h:438-497): strides and padding as well
CONV_SPARSE_PARAMS = ("conv_kh", "conv_kw", "conv_sh", "conv_sw", "conv_padh", "conv_padw", "conv_ih", "conv_iw", "conv_ic",
                      "conv_oh", "conv_ow", "conv_oc")


@dataclass
class Pop:
    name: str
    model: str                      # "lif" | "izh" | "ssa"
    n: int
    params: Dict[str, float] = field(default_factory=dict)
    vars: Dict[str, np.ndarray] = field(default_factory=dict)   # V/RefracTime, V/U, startSpike/endSpike
    spike_times: Optional[np.ndarray] = None                    # ssa only (fp32, ms)


@dataclass
class CurrentSource:
    name: str
    model: str                      # "dc" | "noise" | "poisson_exp" (params weight [nA], tauSyn [ms], rate [Hz])
    pop: str
    amp: float = 0.0
    params: Dict[str, float] = field(default_factory=dict)
    noise: Optional[np.ndarray] = None   # fp32 [steps, n] for "noise"


@dataclass
class Syn:
    name: str
    src: str
    trg: str
    matrix: str = "sparse"          # "sparse" | "conv2d" | "dense" | "bitmask"
    wum: str = "static"             # "static" | "static_delay" | "stdp_trace" | "stdp_additive" (built-in STDP) | "static_const" (one weight, wum_params["g"])
                                    # | "static_reverse" (addToPre(g): the row's weights go back to the spiking neuron)
                                    # | "static_graded" (spike-like events, wum_params["Epre"], ["Vslope"]; source must have a V)
    wum_params: Dict[str, float] = field(default_factory=dict)
    psm: str = "expcurr"            # "expcurr" | "deltacurr"
    tau: float = 5.0
    row_stride: int = 0
    row_length: Optional[np.ndarray] = None   # uint32 [numPre]
    ind: Optional[np.ndarray] = None          # uint32 [numPre, rowStride]
    g: Optional[np.ndarray] = None            # fp32 [numPre, rowStride], dense [numPre, numPost], or kernel [kh,kw,ic,oc]
    gp: Optional[np.ndarray] = None           # bitmask: uint32 words, bit idPre*rowStride + idPost, most significant bit first
    d: Optional[np.ndarray] = None            # uint8 [numPre, rowStride]
    max_den_delay: int = 0
    hint_pre: bool = False
    col_stride: int = 0             # longest column (plastic projections); 0 = let the executor size it
    threads_per_spike: int = 1
    axonal_delay_steps: int = 0     # spikes reach the projection this many timesteps late (SynapseGroup::setAxonalDelaySteps)
    conv: Dict[str, int] = field(default_factory=dict)
    # matrix == "procedural": connect = (snippet, params) of a built-in connectivity snippet, g_init = (snippet, params) of the
    # weight initialisation snippet (or wum "static_const"); nothing is stored.  matrix == "sparse_init": the same two
    # snippets initialise a stored SPARSE matrix (on the host, or on the device where the executor is asked to)
    connect: Optional[tuple] = None
    g_init: Optional[tuple] = None

    @property
    def num_synapses(self):
        if self.matrix == "bitmask":
            return int(np.unpackbits(np.ascontiguousarray(self.gp).view(np.uint8)).sum())
        if self.matrix in ("procedural", "sparse_init"):
            return 0
        if self.matrix == "dense":
            return int(self.g.size) if self.g is not None else 0
        return int(self.row_length.sum()) if self.row_length is not None else 0


@dataclass
class Custom:
    """A custom update (a function of the model called between steps, Runtime::customUpdate) of the test driver:
    kind "decay" (per neuron: V of population `target` towards params rest by params factor, counts its calls),
    "neuron_reduce" (sum and maximum of V over the population, per batch), "wu_decay" (per synapse of projection `target`:
    g *= factor, accumulated), "batch_reduce" (sum and maximum of g over batches), "transpose" (g of DENSE projection
    `target` transposed into g of DENSE projection `target2`); custom connectivity updates of SPARSE projection `target`:
    "prune" (removes synapses with g < params threshold, counting per row) and "sprout" (adds one synapse per row and call
    where there is room, weight params weight)."""
    name: str
    group: str                      # update group: everything in a group runs in one call
    kind: str
    target: str
    target2: str = ""
    params: Dict[str, float] = field(default_factory=dict)


@dataclass
class Net:
    name: str
    dt: float
    steps: int
    pops: List[Pop] = field(default_factory=list)
    css: List[CurrentSource] = field(default_factory=list)
    syns: List[Syn] = field(default_factory=list)
    fuse_psm: bool = False
    seed: int = 0
    # parameters changed while the model runs (setParamDynamic + Runtime::setDynamicParamValue):
    # (kind, group, parameter, step, value) with kind in neuron | cs | wu | ps; the value holds from `step` on
    dynamic: List[tuple] = field(default_factory=list)
    precision: str = "float"        # "double": ModelSpec::setPrecision(Type::Double); the netspec's arrays and the dumps stay fp32
    customs: List[Custom] = field(default_factory=list)
    custom_calls: List[tuple] = field(default_factory=list)     # (update group, every n steps): called after steps n, 2n, ...

    def pop(self, name):
        return next(p for p in self.pops if p.name == name)

    def syn(self, name):
        return next(s for s in self.syns if s.name == name)

    def input_digest(self):
        """SHA-1 over every input array; stored beside golden outputs to detect generator drift."""
        h = hashlib.sha1()
        for p in self.pops:
            for k in sorted(p.vars):
                h.update(np.ascontiguousarray(p.vars[k]).tobytes())
            if p.spike_times is not None:
                h.update(np.ascontiguousarray(p.spike_times).tobytes())
        for c in self.css:
            if c.noise is not None:
                h.update(np.ascontiguousarray(c.noise).tobytes())
        for s in self.syns:
            for a in (s.row_length, s.ind, s.g, s.d, s.gp):
                if a is not None:
                    h.update(np.ascontiguousarray(a).tobytes())
        for d in self.dynamic:
            h.update(repr(tuple(d)).encode())
        if self.precision != "float":
            h.update(self.precision.encode())
        for c in self.customs:
            h.update(repr((c.name, c.group, c.kind, c.target, c.target2, sorted(c.params.items()))).encode())
        for c in self.custom_calls:
            h.update(repr(tuple(c)).encode())
        return h.hexdigest()


def ragged_from_lists(n_pre, pre, post, stride=None, sort=True):
    """Build (rowLength, ind[numPre,stride], order) from COO lists the way
    pygenn/genn_groups.py:434-470 does: lexsort by (pre, post), stride = longest row."""
    pre = np.asarray(pre, dtype=np.int64)
    post = np.asarray(post, dtype=np.int64)
    order = np.lexsort((post, pre)) if sort else np.argsort(pre, kind="stable")
    pre_s, post_s = pre[order], post[order]
    row_length = np.bincount(pre_s, minlength=n_pre).astype(np.uint32)
    stride = int(stride if stride is not None else max(1, row_length.max(initial=0)))
    starts = np.concatenate(([0], np.cumsum(row_length)[:-1])).astype(np.int64)
    within = np.arange(len(pre_s), dtype=np.int64) - starts[pre_s]
    ind = np.zeros((n_pre, stride), dtype=np.uint32)
    ind[pre_s, within] = post_s
    return row_length, ind, order, (pre_s, within)


def write_netspec(net: Net, path: str):
    """Write the directory format read by oracle/ref_driver.cc."""
    os.makedirs(path, exist_ok=True)
    lines = [f"model {net.name}", f"dt {net.dt!r}", f"steps {net.steps}", f"fuse_psm {int(net.fuse_psm)}"]
    snap = getattr(net, "snap", 0)
    lines.append(f"snap {snap}")
    if getattr(net, "batch_size", 1) != 1:
        lines.append(f"batch {int(net.batch_size)}")
    if net.precision != "float":
        lines.append(f"precision {net.precision}")
    if any(s.matrix in ("procedural", "sparse_init") or s.g_init is not None for s in net.syns) or any(c.model == "poisson_exp" for c in net.css) or any(p.model == "poisson" for p in net.pops) \
            or any(s.wum == "stochastic" for s in net.syns):
        lines.append(f"seed {int(net.seed)}")        # procedural matrices and Poisson sources draw from the model's seed
    for kind, group, param, step, value in net.dynamic:
        lines.append(f"dynamic {kind} {group} {param} {int(step)} {float(value)!r}")
    for p in net.pops:
        if p.model == "lif":
            ps = " ".join(repr(float(p.params[k])) for k in LIF_PARAMS)
        elif p.model == "lif_init":   # LIF whose V is drawn by an initialisation snippet (Uniform[Vmin, Vmax)), RefracTime constant 0
            ps = " ".join(repr(float(p.params[k])) for k in LIF_PARAMS + ("Vmin", "Vmax"))
        elif p.model == "lifa":       # LIF with an adaptation variable: a model of the test driver, not a built-in one
            ps = " ".join(repr(float(p.params[k])) for k in LIF_PARAMS + ("TauA", "dA"))
        elif p.model == "izh":
            ps = " ".join(repr(float(p.params[k])) for k in IZH_PARAMS)
        elif p.model == "poisson":    # the built-in Poisson neuron (neuronModels.h:307-325): draws random numbers while it runs
            ps = repr(float(p.params["rate"]))
        else:
            ps = ""
        lines.append(f"pop {p.name} {p.model} {p.n} {ps}".rstrip())
        for k, v in p.vars.items():
            suffix = "u32" if v.dtype == np.uint32 else "f32"
            np.ascontiguousarray(v).tofile(os.path.join(path, f"{p.name}.{k}.{suffix}"))
        if p.spike_times is not None:
            np.ascontiguousarray(p.spike_times, dtype=np.float32).tofile(os.path.join(path, f"{p.name}.spikeTimes.f32"))
    for c in net.css:
        if c.model == "poisson_exp":
            lines.append(f"cs {c.name} poisson_exp {c.pop} {float(c.params['weight'])!r} {float(c.params['tauSyn'])!r} {float(c.params['rate'])!r}")
        elif c.model == "dc":
            lines.append(f"cs {c.name} dc {c.pop} {float(c.amp)!r}")
        else:
            lines.append(f"cs {c.name} noise {c.pop}")
            np.ascontiguousarray(c.noise, dtype=np.float32).tofile(os.path.join(path, f"{c.name}.noise.f32"))
    for s in net.syns:
        if s.matrix == "sparse":
            head = f"syn {s.name} sparse {s.src} {s.trg} {s.row_stride}"
            np.ascontiguousarray(s.row_length, dtype=np.uint32).tofile(os.path.join(path, f"{s.name}.rowLength.u32"))
            np.ascontiguousarray(s.ind, dtype=np.uint32).tofile(os.path.join(path, f"{s.name}.ind.u32"))
        elif s.matrix in ("dense", "dense_init"):
            head = f"syn {s.name} {s.matrix} {s.src} {s.trg}"
        elif s.matrix == "sparse_init" and s.connect[0] == "Conv2D":
            head = f"syn {s.name} conv2d_sparse {s.src} {s.trg} " + " ".join(str(int(s.connect[1][k])) for k in CONV_SPARSE_PARAMS)
        elif s.matrix in ("procedural", "sparse_init"):
            snippet, params = s.connect
            value = params["num"] if snippet in ("FixedNumberPostWithReplacement", "FixedNumberPreWithReplacement") else repr(float(params["prob"]))
            head = f"syn {s.name} {s.matrix} {s.src} {s.trg} {snippet} {value}"
        elif s.matrix == "bitmask":
            head = f"syn {s.name} bitmask {s.src} {s.trg}"
            np.ascontiguousarray(s.gp, dtype=np.uint32).tofile(os.path.join(path, f"{s.name}.gp.u32"))
        else:
            head = f"syn {s.name} conv2d {s.src} {s.trg} " + " ".join(str(int(s.conv[k])) for k in CONV_PARAMS)
        # DENSE with weights from a snippet, never stored; "dense_init": stored, and a kernel whose entries a snippet draws
        regenerated = (s.matrix in ("dense", "dense_init", "conv2d") and s.wum == "static" and s.g_init is not None)
        if s.wum != "static_const" and s.matrix not in ("procedural", "sparse_init") and not regenerated:
            np.ascontiguousarray(s.g, dtype=np.float32).tofile(os.path.join(path, f"{s.name}.g.f32"))
        if s.matrix == "sparse_init" and s.wum == "static" and s.g_init[0] == "Kernel":
            # every weight is an entry of the kernel ([kh][kw][ic][oc]), named by the synapse's position in it
            np.ascontiguousarray(s.g_init[1]["kernel"], dtype=np.float32).tofile(os.path.join(path, f"{s.name}.kernel.f32"))
            w = "static_kernel"
        elif (s.matrix in ("procedural", "sparse_init") or regenerated) and s.wum == "static":
            snippet, params = s.g_init
            order = {"Constant": ("constant",), "Uniform": ("min", "max"), "Normal": ("mean", "sd")}[snippet]
            w = f"static_init {snippet} " + " ".join(repr(float(params[k])) for k in order)
        elif s.wum in ("static", "static_reverse", "timing_copy", "prev_timing"):
            w = s.wum
        elif s.wum == "static_const":
            w = f"static_const {float(s.wum_params['g'])!r}"
        elif s.wum == "static_delay":
            w = f"static_delay {s.max_den_delay}"
            np.ascontiguousarray(s.d, dtype=np.uint8).tofile(os.path.join(path, f"{s.name}.d.u8"))
        elif s.wum in ("stdp_trace", "stdp_additive"):
            w = ("stdp" if s.wum == "stdp_additive" else s.wum) + " " + " ".join(repr(float(s.wum_params[k])) for k in STDP_PARAMS)
        elif s.wum == "static_graded":
            w = f"static_graded {float(s.wum_params['Epre'])!r} {float(s.wum_params['Vslope'])!r}"
        elif s.wum == "stochastic":        # a model of the test driver that draws a random number per synaptic event
            w = f"stochastic {float(s.wum_params['pRelease'])!r}"
        elif s.wum == "post_event":        # a model of the test driver with postsynaptic spike-like events (condition on the target's V)
            w = f"post_event {float(s.wum_params['Vmid'])!r} {float(s.wum_params['back'])!r}"
        elif s.wum == "leaky_graded":      # a model of the test driver with synapse dynamics code (runs for every synapse every step)
            w = f"leaky_graded {float(s.wum_params['Vmid'])!r} {float(s.wum_params['decay'])!r}"
        else:
            raise ValueError(s.wum)
        psm = f"expcurr {float(s.tau)!r}" if s.psm == "expcurr" else "deltacurr"
        opts = (" hint_pre" if s.hint_pre else "") + (f" tps {s.threads_per_spike}" if s.threads_per_spike > 1 else "")
        if s.axonal_delay_steps:
            opts += f" axonal_delay {int(s.axonal_delay_steps)}"
        if s.wum in ("stdp_trace", "stdp_additive", "timing_copy", "prev_timing", "post_event"):
            mask = np.arange(s.row_stride)[None, :] < s.row_length[:, None]
            col = s.col_stride or int(np.bincount(s.ind[mask], minlength=net.pop(s.trg).n).max())
            opts += f" col_stride {max(1, col)}"
        lines.append(f"{head} {w} {psm}{opts}")
    for c in net.customs:
        order = {"decay": ("rest", "factor"), "wu_decay": ("factor",), "prune": ("threshold",), "sprout": ("weight",)}.get(c.kind, ())
        lines.append(" ".join([f"custom {c.name} {c.group} {c.kind} {c.target}"] + ([c.target2] if c.kind == "transpose" else [])
                              + [repr(float(c.params[k])) for k in order]))
    for group, every in net.custom_calls:
        lines.append(f"custom_call {group} {int(every)}")
    with open(os.path.join(path, "net.txt"), "w") as f:
        f.write("\n".join(lines) + "\n")
