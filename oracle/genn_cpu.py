"""TEST INFRASTRUCTURE — binding and builder for the CPU oracle (oracle/genn_cpu.c).

Only tests/, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of bench.py may import
this module.  It builds the oracle with gcc (``-O3 -ffp-contract=off``, no fast-math: the flags
under which the reference's generated C++ is bit-identical to its default unoptimised build)
and constructs an oracle network from a :class:`genn_amd.netspec.Net`, deriving every fp32
constant on its own, the way the reference does: literals go double -> "%.9e" -> float
(src/genn/genn/type.cc:329-350) when equal across a merged group, plain double -> float
casts otherwise (include/genn/genn/code_generator/environment.h:483-511).
"""
import ctypes as C
import math
import os
import subprocess
from decimal import Decimal

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
LIB = os.path.join(HERE, "libgenn_cpu_oracle.so")
SRC = os.path.join(HERE, "genn_cpu.c")

GC_LIF, GC_IZH, GC_SSA = 0, 1, 2
GC_EXPCURR, GC_DELTACURR = 0, 1
GC_STATIC, GC_STATIC_DELAY, GC_STDP_TRACE, GC_STATIC_GRADED, GC_STATIC_REVERSE, GC_STDP_ADDITIVE = 0, 1, 2, 3, 4, 5
GC_CS_DC, GC_CS_NOISE, GC_CS_POISSON_EXP = 0, 1, 2


def build(force=False):
    if force or not os.path.exists(LIB) or os.path.getmtime(LIB) < os.path.getmtime(SRC):
        subprocess.check_call(["gcc", "-O3", "-ffp-contract=off", "-fno-fast-math", "-shared", "-fPIC", "-o", LIB, SRC, "-lm"])
    return LIB


_lib = None


def lib():
    global _lib
    if _lib is None:
        l = C.CDLL(build())
        vp, u32, u64, f32, i32 = C.c_void_p, C.c_uint32, C.c_uint64, C.c_float, C.c_int
        l.gc_create.restype = vp; l.gc_create.argtypes = [f32, u64]
        l.gc_add_pop.restype = i32; l.gc_add_pop.argtypes = [vp, i32, u32, vp, i32, vp, vp, vp]
        l.gc_add_psm.restype = i32; l.gc_add_psm.argtypes = [vp, i32, i32, f32, f32, u32]
        l.gc_add_cs.restype = i32; l.gc_add_cs.argtypes = [vp, i32, i32, f32, vp, u64]
        l.gc_add_cs_poisson_exp.restype = i32; l.gc_add_cs_poisson_exp.argtypes = [vp, i32, f32, f32, f32, u64, u32, u32, vp]
        l.gc_philox4x32.restype = None; l.gc_philox4x32.argtypes = [u32] * 6 + [vp]
        l.gc_cs_current.restype = vp; l.gc_cs_current.argtypes = [vp, i32, i32]
        l.gc_add_syn_sparse.restype = i32; l.gc_add_syn_sparse.argtypes = [vp, i32, i32, i32, i32, u32, vp, vp, vp, vp, i32]
        l.gc_set_stdp_additive.restype = None; l.gc_set_stdp_additive.argtypes = [vp, i32, f32, f32, f32, f32, f32, f32, u32]
        l.gc_set_stdp_trace.restype = None; l.gc_set_stdp_trace.argtypes = [vp, i32, f32, f32, f32, f32, f32, f32, u32]
        l.gc_add_syn_conv2d.restype = i32; l.gc_add_syn_conv2d.argtypes = [vp, i32, i32, i32, vp, vp]
        l.gc_set_delay_slots.restype = None; l.gc_set_delay_slots.argtypes = [vp, i32, u32]
        l.gc_set_axonal_delay.restype = None; l.gc_set_axonal_delay.argtypes = [vp, i32, u32]
        l.gc_add_syn_dense.restype = i32; l.gc_add_syn_dense.argtypes = [vp, i32, i32, i32, vp, C.c_float]
        l.gc_add_syn_bitmask.restype = i32; l.gc_add_syn_bitmask.argtypes = [vp, i32, i32, i32, vp, u32, C.c_float]
        l.gc_build_remap.restype = None; l.gc_build_remap.argtypes = [vp, i32]
        l.gc_step.restype = None; l.gc_step.argtypes = [vp]
        l.gc_advance.restype = None; l.gc_advance.argtypes = [vp]
        l.gc_update_synapses.restype = None; l.gc_update_synapses.argtypes = [vp, f32]
        l.gc_update_neurons.restype = None; l.gc_update_neurons.argtypes = [vp, f32, u32]
        l.gc_run.restype = None; l.gc_run.argtypes = [vp, u64]
        l.gc_spike_count.restype = u32; l.gc_spike_count.argtypes = [vp, i32]
        for name in ("gc_spikes", "gc_start_spike", "gc_record", "gc_pre_trace", "gc_post_trace", "gc_spike_time"):
            getattr(l, name).restype = vp; getattr(l, name).argtypes = [vp, i32]
        l.gc_var.restype = vp; l.gc_var.argtypes = [vp, i32, i32]
        l.gc_out_post.restype = vp; l.gc_out_post.argtypes = [vp, i32, i32]
        l.gc_den_delay.restype = vp; l.gc_den_delay.argtypes = [vp, i32, i32]
        l.gc_den_delay_ptr.restype = u32; l.gc_den_delay_ptr.argtypes = [vp, i32, i32]
        for name in ("gc_syn_g", "gc_col_length", "gc_remap"):
            getattr(l, name).restype = vp; getattr(l, name).argtypes = [vp, i32]
        l.gc_syn_events.restype = u64; l.gc_syn_events.argtypes = [vp, i32]
        l.gc_set_static_graded.restype = None; l.gc_set_static_graded.argtypes = [vp, i32, f32, f32]
        l.gc_set_static_reverse.restype = None; l.gc_set_static_reverse.argtypes = [vp, i32]
        l.gc_out_pre.restype = vp; l.gc_out_pre.argtypes = [vp, i32]
        l.gc_event_count.restype = u32; l.gc_event_count.argtypes = [vp, i32, i32]
        l.gc_events.restype = vp; l.gc_events.argtypes = [vp, i32, i32]
        l.gc_event_record.restype = vp; l.gc_event_record.argtypes = [vp, i32, i32]
        l.gc_syn_event_queue.restype = i32; l.gc_syn_event_queue.argtypes = [vp, i32]
        l.gc_timestep.restype = u64; l.gc_timestep.argtypes = [vp]
        l.gc_destroy.restype = None; l.gc_destroy.argtypes = [vp]
        _lib = l
    return _lib


def literal_f32(x):
    """double -> '%.9e' -> nearest float (ties to even), exactly, via decimal arithmetic."""
    x = float(x)
    if x == 0.0:
        return np.float32(0.0)
    exact = Decimal("%.9e" % x)
    guess = np.float32(float(exact))
    cands = [np.nextafter(guess, np.float32(-np.inf)), guess, np.nextafter(guess, np.float32(np.inf))]
    best = min(cands, key=lambda c: (abs(Decimal(float(c)) - exact), int(np.float32(c).view(np.uint32)) & 1))
    return np.float32(best)


def _round_group(vals):
    if all(float(v) == float(vals[0]) for v in vals):
        return [literal_f32(v) for v in vals]
    return [np.float32(float(v)) for v in vals]


def _as(a, dtype):
    return np.ascontiguousarray(a, dtype=dtype)


class OracleNet:
    """The oracle's view of a Net.  ``max_col`` maps projection name -> column stride."""

    def __init__(self, net, num_recording_timesteps=0, col_stride=None, batch_index=0):
        self.l = lib()
        self.net = net
        self.keep = []               # arrays the C side borrows
        self.num_rec = num_recording_timesteps
        self.h = self.l.gc_create(C.c_float(literal_f32(net.dt)), num_recording_timesteps)
        self.pop_id, self.syn_id, self.psm_id = {}, {}, {}
        dt = net.dt
        in_syn = {p.name: [s for s in net.syns if s.trg == p.name] for p in net.pops}
        out_syn = {p.name: [s for s in net.syns if s.src == p.name] for p in net.pops}

        # fused postsynaptic models per target population
        fused = {}
        for p in net.pops:
            groups = []
            # the reference fuses from the last projection added to the first (neuronGroup.cc:41-96)
            for s in reversed(in_syn[p.name]):
                key = (s.psm, s.tau if s.psm == "expcurr" else None, s.max_den_delay if s.wum == "static_delay" else 0)
                hit = next((g for g in groups if net.fuse_psm and g[0] == key), None)
                if hit is None:
                    groups.append((key, [s]))
                else:
                    hit[1].append(s)
            # children sorted by structure only; equal structure keeps creation order
            groups.sort(key=lambda g: (g[0][0], g[0][2]))
            fused[p.name] = groups

        def merge_key(p):
            cs = tuple(c.model for c in net.css if c.pop == p.name)
            psm = tuple((g[0][0], g[0][2]) for g in fused[p.name])
            pre = any(s.wum == "stdp_trace" for s in out_syn[p.name])
            post = any(s.wum == "stdp_trace" for s in in_syn[p.name])
            slots = max([s.axonal_delay_steps for s in out_syn[p.name]], default=0) + 1
            events = len({float(s.wum_params["Epre"]) for s in out_syn[p.name] if s.wum == "static_graded"})
            reverse = sum(s.wum == "static_reverse" for s in out_syn[p.name])
            return (p.model, psm, cs, pre, post, slots, events, reverse)

        merged = {}
        for p in net.pops:
            merged.setdefault(merge_key(p), []).append(p)

        lif_derive = lambda q: [q["Ioffset"], q["TauM"] / q["C"], q["Vrest"], math.exp(-dt / q["TauM"]), q["Vthresh"], q["Vreset"], q["TauRefrac"]]
        params = {}
        for members in merged.values():
            if members[0].model == "lif":
                cols = [_round_group(list(c)) for c in zip(*[lif_derive(p.params) for p in members])]
            elif members[0].model == "izh":
                cols = [_round_group(list(c)) for c in zip(*[[p.params[k] for k in "abcd"] for p in members])]
            else:
                cols = []
            for k, p in enumerate(members):
                params[p.name] = np.array([c[k] for c in cols], dtype=np.float32)

        for p in net.pops:
            model = {"lif": GC_LIF, "izh": GC_IZH, "ssa": GC_SSA}[p.model]
            if p.model == "ssa":
                v0, v1 = _as(p.vars["startSpike"], np.uint32), _as(p.vars["endSpike"], np.uint32)
                st = _as(p.spike_times if p.spike_times.size else np.zeros(1), np.float32)
                self.keep.append(st)
                stp = st.ctypes.data
            else:
                names = ("V", "RefracTime") if p.model == "lif" else ("V", "U")
                v0, v1 = _as(p.vars[names[0]], np.float32), _as(p.vars[names[1]], np.float32)
                stp = None
            pr = params[p.name]
            self.pop_id[p.name] = self.l.gc_add_pop(self.h, model, p.n, pr.ctypes.data if pr.size else None, pr.size,
                                                    v0.ctypes.data, v1.ctypes.data, stp)

        # delay slots: longest axonal delay among a population's outgoing projections, plus one
        for p in net.pops:
            slots = max([s.axonal_delay_steps for s in out_syn[p.name]], default=0) + 1
            if slots > 1:
                self.l.gc_set_delay_slots(self.h, self.pop_id[p.name], slots)

        # postsynaptic-model children with merged-group rounding, matched by child index
        for members in merged.values():
            for m in range(len(fused[members[0].name])):
                keys = [fused[p.name][m][0] for p in members]
                if keys[0][0] == "expcurr":
                    decay = _round_group([math.exp(-dt / k[1]) for k in keys])
                    init = _round_group([(k[1] * (1.0 - math.exp(-dt / k[1]))) * (1.0 / dt) for k in keys])
                for j, p in enumerate(members):
                    key, syns = fused[p.name][m]
                    if key[0] == "expcurr":
                        pid = self.l.gc_add_psm(self.h, self.pop_id[p.name], GC_EXPCURR, C.c_float(init[j]), C.c_float(decay[j]), key[2])
                    else:
                        pid = self.l.gc_add_psm(self.h, self.pop_id[p.name], GC_DELTACURR, 0.0, 0.0, key[2])
                    for s in syns:
                        self.psm_id[s.name] = pid
            css = [[c for c in net.css if c.pop == p.name] for p in members]
            for ci in range(len(css[0])):
                if css[0][ci].model == "dc":
                    amps = _round_group([c[ci].amp for c in css])
                if css[0][ci].model == "poisson_exp":
                    # derived parameters of the snippet (currentSourceModels.h:123-128), rounded like any merged-group constant
                    q = [c[ci].params for c in css]
                    decay = _round_group([math.exp(-dt / x["tauSyn"]) for x in q])
                    init = _round_group([x["weight"] * (1.0 - math.exp(-dt / x["tauSyn"])) * (x["tauSyn"] / dt) for x in q])
                    lam = _round_group([math.exp(-(x["rate"] / 1000.0) * dt) for x in q])
                for j, p in enumerate(members):
                    c = css[j][ci]
                    if c.model == "poisson_exp":
                        stream = 1000 + sorted(x.name for x in net.css).index(c.name)      # by place in the name-ordered list of the model's sources
                        zero = np.zeros(p.n, np.float32)
                        self.l.gc_add_cs_poisson_exp(self.h, self.pop_id[p.name], C.c_float(init[j]), C.c_float(decay[j]), C.c_float(lam[j]),
                                                     net.seed, stream, batch_index * p.n, zero.ctypes.data)
                        self.cs_id = getattr(self, "cs_id", {})
                        self.cs_id[c.name] = (p.name, ci)
                        continue
                    if c.model == "dc":
                        self.l.gc_add_cs(self.h, self.pop_id[p.name], GC_CS_DC, C.c_float(amps[j]), None, 0)
                    else:
                        a = _as(c.noise, np.float32)
                        self.keep.append(a)
                        self.l.gc_add_cs(self.h, self.pop_id[p.name], GC_CS_NOISE, 0.0, a.ctypes.data, a.size // p.n)

        for s in net.syns:
            src, trg = self.pop_id[s.src], self.pop_id[s.trg]
            if s.matrix == "sparse":
                rl, ind = _as(s.row_length, np.uint32), _as(s.ind, np.uint32)
                # StaticPulseConstantWeight (weightUpdateModels.h:202-213) adds its parameter g for every synapse: same loop,
                # same value everywhere
                g = np.full(ind.shape, literal_f32(s.wum_params["g"]), np.float32) if s.wum == "static_const" else _as(s.g, np.float32)
                d = _as(s.d, np.uint8) if s.d is not None else None
                self.keep += [rl, ind, g, d]
                wum = {"static": GC_STATIC, "static_const": GC_STATIC, "static_delay": GC_STATIC_DELAY, "stdp_trace": GC_STDP_TRACE,
                       "static_graded": GC_STATIC_GRADED, "static_reverse": GC_STATIC_REVERSE, "stdp_additive": GC_STDP_ADDITIVE}[s.wum]
                sid = self.l.gc_add_syn_sparse(self.h, src, trg, self.psm_id[s.name], wum, s.row_stride, rl.ctypes.data, ind.ctypes.data,
                                               g.ctypes.data, d.ctypes.data if d is not None else None, int(s.wum in ("stdp_trace", "stdp_additive")))
                if s.wum == "static_reverse":
                    self.l.gc_set_static_reverse(self.h, sid)
                if s.wum == "static_graded":
                    # Epre and Vslope are literals when every graded projection has the same value, struct fields otherwise
                    graded = [x for x in net.syns if x.wum == "static_graded" and x.matrix == "sparse"]
                    k = graded.index(s)
                    self.l.gc_set_static_graded(self.h, sid, C.c_float(_round_group([x.wum_params["Epre"] for x in graded])[k]),
                                                C.c_float(_round_group([x.wum_params["Vslope"] for x in graded])[k]))
                if s.wum in ("stdp_trace", "stdp_additive"):
                    q = s.wum_params
                    stride = (col_stride or {}).get(s.name)
                    if stride is None:
                        mask = np.arange(s.row_stride)[None, :] < rl[:, None]
                        stride = int(np.bincount(ind.reshape(len(rl), -1)[mask], minlength=net.pop(s.trg).n).max())
                if s.wum == "stdp_additive":
                    # the six parameters are literals in the generated code (one plastic projection per merged group)
                    self.l.gc_set_stdp_additive(self.h, sid, *(C.c_float(literal_f32(q[k])) for k in ("tauPlus", "tauMinus", "aPlus", "aMinus", "wMin", "wMax")),
                                                max(1, stride))
                    self.l.gc_build_remap(self.h, sid)
                    self.col_stride = getattr(self, "col_stride", {})
                    self.col_stride[s.name] = max(1, stride)
                if s.wum == "stdp_trace":
                    self.l.gc_set_stdp_trace(self.h, sid, C.c_float(literal_f32(q["aPlus"])), C.c_float(literal_f32(q["aMinus"])),
                                             C.c_float(literal_f32(q["wMin"])), C.c_float(literal_f32(q["wMax"])),
                                             C.c_float(literal_f32(math.exp(-dt / q["tauPlus"]))),
                                             C.c_float(literal_f32(math.exp(-dt / q["tauMinus"]))), max(1, stride))
                    self.l.gc_build_remap(self.h, sid)
                    self.col_stride = getattr(self, "col_stride", {})
                    self.col_stride[s.name] = max(1, stride)
            elif s.matrix == "dense":
                g = _as(s.g, np.float32) if s.g is not None else None
                self.keep.append(g)
                sid = self.l.gc_add_syn_dense(self.h, src, trg, self.psm_id[s.name], g.ctypes.data if g is not None else None,
                                              C.c_float(literal_f32(s.wum_params.get("g", 0.0))))
            elif s.matrix == "bitmask":
                gp = _as(s.gp, np.uint32)
                self.keep.append(gp)
                sid = self.l.gc_add_syn_bitmask(self.h, src, trg, self.psm_id[s.name], gp.ctypes.data, s.row_stride,
                                                C.c_float(literal_f32(s.wum_params["g"])))
            else:
                conv = np.array([s.conv[k] for k in ("conv_kh", "conv_kw", "conv_ih", "conv_iw", "conv_ic", "conv_oh", "conv_ow", "conv_oc")], dtype=np.int32)
                kern = _as(s.g, np.float32)
                self.keep += [conv, kern]
                sid = self.l.gc_add_syn_conv2d(self.h, src, trg, self.psm_id[s.name], conv.ctypes.data, kern.ctypes.data)
            self.syn_id[s.name] = sid
            if s.axonal_delay_steps:
                self.l.gc_set_axonal_delay(self.h, sid, s.axonal_delay_steps)

    # ---- stepping and state -----------------------------------------------------------------
    def step(self):
        self.l.gc_step(self.h)

    def run(self, steps):
        self.l.gc_run(self.h, steps)

    @property
    def timestep(self):
        return int(self.l.gc_timestep(self.h))

    def update_synapses(self):
        """First half of step(): the runner's updateSynapses(t)."""
        self.l.gc_update_synapses(self.h, C.c_float(np.float32(self.timestep) * np.float32(literal_f32(self.net.dt))))

    def update_neurons(self):
        """Second half of step(): updateNeurons(t, recordingTimestep); advances time."""
        ts = self.timestep
        self.l.gc_update_neurons(self.h, C.c_float(np.float32(ts) * np.float32(literal_f32(self.net.dt))),
                                 (ts % self.num_rec) if self.num_rec else 0)
        self.l.gc_advance(self.h)

    def _arr(self, ptr, n, dtype):
        if not ptr or n == 0:
            return np.zeros(0, dtype=dtype)
        return np.ctypeslib.as_array(C.cast(ptr, C.POINTER(np.ctypeslib.as_ctypes_type(dtype))), shape=(n,))

    def spikes(self, pop):
        n = self.l.gc_spike_count(self.h, self.pop_id[pop])
        return self._arr(self.l.gc_spikes(self.h, self.pop_id[pop]), n, np.uint32).copy()

    def var(self, pop, which):
        return self._arr(self.l.gc_var(self.h, self.pop_id[pop], which), self.net.pop(pop).n, np.float32)

    def start_spike(self, pop):
        return self._arr(self.l.gc_start_spike(self.h, self.pop_id[pop]), self.net.pop(pop).n, np.uint32)

    def out_post(self, syn):
        s = self.net.syn(syn)
        return self._arr(self.l.gc_out_post(self.h, self.pop_id[s.trg], self.psm_id[syn]), self.net.pop(s.trg).n, np.float32)

    def den_delay(self, syn):
        s = self.net.syn(syn)
        return self._arr(self.l.gc_den_delay(self.h, self.pop_id[s.trg], self.psm_id[syn]), self.net.pop(s.trg).n * s.max_den_delay, np.float32)

    def syn_g(self, syn):
        s = self.net.syn(syn)
        return self._arr(self.l.gc_syn_g(self.h, self.syn_id[syn]), self.net.pop(s.src).n * s.row_stride, np.float32)

    def pre_trace(self, pop):
        return self._arr(self.l.gc_pre_trace(self.h, self.pop_id[pop]), self.net.pop(pop).n, np.float32)

    def post_trace(self, pop):
        return self._arr(self.l.gc_post_trace(self.h, self.pop_id[pop]), self.net.pop(pop).n, np.float32)

    def col_length(self, syn):
        s = self.net.syn(syn)
        return self._arr(self.l.gc_col_length(self.h, self.syn_id[syn]), self.net.pop(s.trg).n, np.uint32)

    def remap(self, syn):
        s = self.net.syn(syn)
        return self._arr(self.l.gc_remap(self.h, self.syn_id[syn]), self.net.pop(s.trg).n * self.col_stride[syn], np.uint32)

    def record(self, pop, num_rec):
        n = self.net.pop(pop).n
        return self._arr(self.l.gc_record(self.h, self.pop_id[pop]), num_rec * ((n + 31) // 32), np.uint32)

    def out_pre(self, syn):
        s = self.net.syn(syn)
        return self._arr(self.l.gc_out_pre(self.h, self.syn_id[syn]), self.net.pop(s.src).n, np.float32)

    def cs_current(self, name):
        pop, ci = self.cs_id[name]
        return self._arr(self.l.gc_cs_current(self.h, self.pop_id[pop], ci), self.net.pop(pop).n, np.float32)

    def spike_events(self, syn):
        """The spike-like event queue a graded projection read last / will read next (ids in ascending order)."""
        s = self.net.syn(syn)
        pop, q = self.pop_id[s.src], self.l.gc_syn_event_queue(self.h, self.syn_id[syn])
        return self._arr(self.l.gc_events(self.h, pop, q), self.l.gc_event_count(self.h, pop, q), np.uint32).copy()

    def event_record(self, syn, num_rec):
        """Recorded spike-like events of the queue a graded projection reads: bitfield [num_rec, ceil(n/32)]."""
        s = self.net.syn(syn)
        pop, q = self.pop_id[s.src], self.l.gc_syn_event_queue(self.h, self.syn_id[syn])
        n = self.net.pop(s.src).n
        return self._arr(self.l.gc_event_record(self.h, pop, q), num_rec * ((n + 31) // 32), np.uint32)

    def events(self):
        return sum(self.l.gc_syn_events(self.h, i) for i in self.syn_id.values())

    def close(self):
        if self.h:
            self.l.gc_destroy(self.h)
            self.h = None
