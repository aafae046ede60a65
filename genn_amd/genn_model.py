"""Host side of the MI355X backend: a model description with PyGeNN's surface
(``GeNNModel.add_neuron_population / add_synapse_population / add_current_source / build /
load / step_time``, pygenn/genn_model.py:159-847) for the fixed set of snippets on the hot path,
plus the work the reference's ``Runtime`` does around a generated runner: allocate every array
with the reference's names and sizes (src/genn/genn/runtime/runtime.cc:147-402), push one
merged-group descriptor per group (runtime.h:573-669), and step.

All device work goes through the C ABI in include/genn_mi355x.h; nothing here computes the
simulation on the host.
"""
import ctypes as C
import math
import time
from fractions import Fraction

import numpy as np

from . import _abi

FLT_MAX = np.float32(3.402823466e+38)


# --------------------------------------------------------------------------------------------
# numeric literal handling
# --------------------------------------------------------------------------------------------
def lit32(x):
    """fp32 value of a parameter the reference bakes into generated code as a literal:
    double -> ``%.9e`` text -> correctly rounded float (src/genn/genn/type.cc:329-350)."""
    x = float(x)
    if x == 0.0 or math.isinf(x) or math.isnan(x):
        return np.float32(x)
    text = "%.9e" % x
    exact = Fraction(text)
    c = np.float32(float(text))
    best = None
    for cand in (np.nextafter(c, np.float32(-np.inf)), c, np.nextafter(c, np.float32(np.inf))):
        if not np.isfinite(cand):
            continue
        err = abs(Fraction(float(cand)) - exact)
        even = (int(np.float32(cand).view(np.uint32)) & 1) == 0
        key = (err, 0 if even else 1)
        if best is None or key < best[0]:
            best = (key, cand)
    return np.float32(best[1])


def field32(x):
    """fp32 value of a parameter that is heterogeneous across a merged group and therefore
    travels as a struct field: a plain double->float cast (runtime.h:647-651)."""
    return np.float32(float(x))


def _merge_round(values):
    """Literal rounding when every group of the merged group agrees, field rounding otherwise
    (include/genn/genn/code_generator/environment.h:483-511)."""
    same = all(float(v) == float(values[0]) for v in values)
    return [lit32(v) if same else field32(v) for v in values]


# --------------------------------------------------------------------------------------------
# snippet initialisers with PyGeNN's names (pygenn/genn_model.py init_* helpers)
# --------------------------------------------------------------------------------------------
class _Init:
    def __init__(self, snippet, params=None, vars=None, pre_vars=None, post_vars=None):
        self.snippet = snippet
        self.params = dict(params or {})
        self.vars = dict(vars or {})
        self.pre_vars = dict(pre_vars or {})
        self.post_vars = dict(post_vars or {})


def init_postsynaptic(snippet, params=None, vars=None):
    if snippet not in ("ExpCurr", "DeltaCurr"):
        raise NotImplementedError(f"postsynaptic model {snippet}")
    return _Init(snippet, params, vars)


def init_weight_update(snippet, params=None, vars=None, pre_vars=None, post_vars=None):
    if snippet not in ("StaticPulse", "StaticPulseConstantWeight", "StaticPulseDendriticDelay", "STDPTrace", "STDP", "StaticGraded", "StaticPulseReverse"):
        raise NotImplementedError(f"weight update model {snippet}")
    return _Init(snippet, params, vars, pre_vars, post_vars)


def init_toeplitz_connectivity(snippet, params=None):
    if snippet != "Conv2D":
        raise NotImplementedError(f"toeplitz connectivity {snippet}")
    return _Init(snippet, params)


# initSparseConnectivitySnippet.h:107-370; maximum row length as each snippet's SET_CALC_MAX_ROW_LENGTH_FUNC
_SPARSE_SNIPPETS = ("OneToOne", "FixedProbability", "FixedProbabilityNoAutapse", "FixedNumberPostWithReplacement",
                    "FixedNumberTotalWithReplacement", "FixedNumberPreWithReplacement", "Conv2D")
_CONV2D_PARAMS = ("conv_kh", "conv_kw", "conv_sh", "conv_sw", "conv_padh", "conv_padw", "conv_ih", "conv_iw", "conv_ic",
                  "conv_oh", "conv_ow", "conv_oc")


def init_sparse_connectivity(snippet, params=None):
    """Connectivity built on the device at load() (pygenn.init_sparse_connectivity)."""
    if snippet not in _SPARSE_SNIPPETS:
        raise NotImplementedError(f"sparse connectivity snippet {snippet}")
    return _Init(snippet, params)


def binomial_inverse_cdf(cdf, n, p):
    """GeNN::binomialInverseCDF (src/genn/genn/binomial.cc:37-110): the reference's unit test holds it to scipy's
    binom.ppf (tests/unit/binomial.cc)."""
    from scipy import stats
    return int(stats.binom.ppf(cdf, n, p))


def max_row_length(snippet, params, num_pre, num_post):
    if snippet == "OneToOne":
        return 1
    if snippet in ("FixedProbability", "FixedProbabilityNoAutapse"):
        # initSparseConnectivitySnippet.h:135-142
        return max(1, binomial_inverse_cdf(0.9999 ** (1.0 / num_pre), num_post, float(params["prob"])))
    if snippet == "FixedNumberPostWithReplacement":
        return int(params["num"])
    if snippet == "FixedNumberTotalWithReplacement":
        # :372-381: rows are binomial(num, 1/numPre)
        return max(1, binomial_inverse_cdf(0.9999 ** (1.0 / num_pre), int(params["num"]), 1.0 / num_pre))
    if snippet == "FixedNumberPreWithReplacement":
        # :391-400: a row receives each of the num * numPost draws with probability 1 / numPre
        return max(1, binomial_inverse_cdf(0.9999 ** (1.0 / num_pre), int(params["num"]) * num_post, 1.0 / num_pre))
    if snippet == "Conv2D":
        # :485-491
        kh, kw, sh, sw, oc = (int(params[k]) for k in ("conv_kh", "conv_kw", "conv_sh", "conv_sw", "conv_oc"))
        return -(-kh // sh) * -(-kw // sw) * oc
    raise NotImplementedError(snippet)


class VarInit:
    """Value snippet evaluated on the device at load() (pygenn.init_var; initVarSnippet.h:87-262)."""
    _PARAMS = {"Constant": ("constant",), "Uniform": ("min", "max"), "Normal": ("mean", "sd"),
               "NormalClipped": ("mean", "sd", "min", "max"), "NormalClippedDelay": ("mean", "sd", "min", "max"),
               "Exponential": ("lambda",), "Gamma": ("a", "b"), "Binomial": ("n", "p"),
               # initVarSnippet.h:100-108: the value is an entry of the `kernel` array (an extra global parameter in the
               # reference), which one names the connectivity snippet; only behind Conv2D connectivity here
               "Kernel": ("kernel",)}

    def __init__(self, snippet, params):
        if snippet not in self._PARAMS:
            raise NotImplementedError(f"variable initialisation snippet {snippet}")
        missing = [k for k in self._PARAMS[snippet] if k not in params]
        if missing:
            raise ValueError(f"{snippet}: missing parameter(s) {missing}")
        self.snippet = snippet
        self.params = dict(params)

    def values(self, dt):
        if self.snippet == "Kernel":
            raise NotImplementedError("Kernel variable initialisation is only available behind Conv2D sparse connectivity")
        v = [float(self.params[k]) for k in self._PARAMS[self.snippet]]
        if self.snippet == "NormalClippedDelay":
            v = [x / dt for x in v]          # the snippet's derived parameters (initVarSnippet.h:204-208)
        return v + [0.0] * (4 - len(v))


def init_var(snippet, params=None):
    return VarInit(snippet, params or {})


# --------------------------------------------------------------------------------------------
# device arrays (the reference's Array objects, src/genn/backends/hip/backend.cc:61-236)
# --------------------------------------------------------------------------------------------
class Array:
    def __init__(self, count, dtype, fill=None, device_only=False):
        """``device_only`` arrays (those a device kernel initialises) get their host copy on the first pull."""
        self.dtype = np.dtype(dtype)
        self.count = int(count)
        self._dev = C.c_void_p()
        _abi.check(_abi.load().gennmi_malloc(C.byref(self._dev), self.count * self.dtype.itemsize))
        self._view = None
        if not device_only:
            self._view = np.zeros(self.count, dtype=self.dtype) if fill is None else np.full(self.count, fill, dtype=self.dtype)
            self.push_to_device()

    @property
    def view(self):
        if self._view is None:
            self._view = np.zeros(self.count, dtype=self.dtype)
        return self._view

    @property
    def ptr(self):
        return self._dev.value

    @property
    def values(self):
        return self.view

    def push_to_device(self):
        if self.view.nbytes:
            _abi.check(_abi.load().gennmi_memcpy_to_device(self._dev, self.view.ctypes.data_as(C.c_void_p), self.view.nbytes))

    def pull_from_device(self):
        if self.view.nbytes:
            _abi.check(_abi.load().gennmi_memcpy_from_device(self.view.ctypes.data_as(C.c_void_p), self._dev, self.view.nbytes))
        return self.view

    def pull_slice(self, first, count):
        """Elements first .. first + count - 1 from the device, as a new array (for arrays too large to mirror on the host)."""
        first, count = int(first), int(count)
        if first < 0 or count < 0 or first + count > self.count:
            raise IndexError("slice outside the array")
        out = np.empty(count, dtype=self.dtype)
        if count:
            _abi.check(_abi.load().gennmi_memcpy_from_device(out.ctypes.data_as(C.c_void_p), C.c_void_p(self._dev.value + first * self.dtype.itemsize), out.nbytes))
        return out

    def init_on_device(self, init, seed, stream, dt):
        """Fill from a value snippet (gennmi_init_var); the host copy is not touched."""
        params = (C.c_double * 4)(*init.values(dt))
        _abi.check(_abi.load().gennmi_init_var(self._dev, _abi.ELEMENT_TYPES[self.dtype.name], self.count,
                                               _abi.INIT_SNIPPETS[init.snippet], C.byref(params), seed, stream))

    def copy_on_device(self, src):
        """Device-to-device copy of another fp32 Array of the same length (host views are left alone)."""
        if self.dtype != np.float32 or src.dtype != np.float32 or src.count != self.count:
            raise ValueError("copy_on_device needs two float32 arrays of equal length")
        _abi.check(_abi.load().gennmi_copy_f32(self._dev, src._dev, self.count))

    def free(self):
        if self._dev:
            _abi.load().gennmi_free(self._dev)
            self._dev = C.c_void_p()


class NeuronGroup:
    def __init__(self, model, name, n, neuron, params, vars):
        self._model = model
        self.name = name
        self.num_neurons = int(n)
        self.neuron = neuron
        self.params = dict(params)
        self.var_init = dict(vars)
        self.vars = {}
        self.extra_global_params = {}
        self.current_sources = []
        self.in_syn = []
        self.out_syn = []
        self.spike_recording_enabled = False
        self.spike_event_recording_enabled = False
        self.fused_psm = []          # list of lists of SynapseGroup sharing one outPost
        self.pre_trace_owner = None
        self.post_trace_owner = None
        self.needs_spike_time = False
        self.num_delay_slots = 1     # longest axonal delay of the outgoing projections + 1, set by build()
        self.pre_output_syn = []     # outgoing projections whose code calls addToPre
        self.event_thresholds = []   # one spike-like event queue per distinct threshold of the outgoing graded projections

    @property
    def size(self):
        return self.num_neurons

    def set_extra_global_param(self, name, value):
        self.extra_global_params[name] = np.ascontiguousarray(value)

    @property
    def spike_recording_data(self):
        """[(times, ids)] per batch, decoded from the recordSpk bitfield (runtime.cc:855-913)."""
        return self._model._decode_recording(self)

    @property
    def current_spikes(self):
        """Spike queue written by the last step: ids in ascending order (per batch)."""
        # with axonal delay the queue is a ring of slots; the last step wrote slot timestep % slots (pygenn's current_spikes
        # reads spkQuePtr the same way, genn_groups.py)
        slots, B = self.num_delay_slots, self._model.batch_size
        slot = self._model.timestep % slots
        cnt = self.vars["spkCnt"].pull_from_device().reshape(B, slots)[:, slot].copy()
        spk = self.vars["spk"].pull_from_device().reshape(B, slots, self.num_neurons)[:, slot]
        return [spk[b, :cnt[b]].copy() for b in range(B)]


class CurrentSource:
    def __init__(self, name, kind, pop, params):
        self.name = name
        self.kind = kind
        self.pop = pop
        self.params = dict(params)
        self.extra_global_params = {}
        self.vars = {}
        self.stream = None          # PoissonExp: generator stream (the next free one of the model unless set)

    def set_extra_global_param(self, name, value):
        self.extra_global_params[name] = np.ascontiguousarray(value, dtype=np.float32)


class SynapseGroup:
    def __init__(self, model, name, matrix_type, src, trg, wu, ps, conn):
        self._model = model
        self.name = name
        self.matrix_type = matrix_type
        self.src = src
        self.trg = trg
        self.wu = wu
        self.ps = ps
        self.conn = conn
        self.vars = {}
        self.max_dendritic_delay_timesteps = 1
        self.parallelism_hint = "POSTSYNAPTIC"
        self.num_threads_per_spike = 1
        self.axonal_delay_steps = 0
        self.row_stride = 0
        self.col_stride = 0
        self.row_length_host = None
        self.ind_host = None
        self.var_host = {}
        self.gp_host = None
        self.procedural_streams = None
        self.fused_ps_target = self

    # pygenn/genn_groups.py:434-470
    def set_sparse_connections(self, pre_indices, post_indices):
        pre = np.asarray(pre_indices, dtype=np.int64)
        post = np.asarray(post_indices, dtype=np.int64)
        if self.matrix_type == "BITMASK":
            # one bit per pair, gid = idPre*rowStride + idPost with the row stride padded to 32, most significant bit of a
            # word first (single_threaded_cpu/backend.cc:1393-1404, 2003-2006)
            stride = (self.trg.num_neurons + 31) // 32 * 32
            bits = np.zeros(self.src.num_neurons * stride, dtype=np.uint8)
            bits[pre * stride + post] = 1
            self.gp_host = np.packbits(bits, bitorder="big").view(">u4").astype(np.uint32)
            self.row_stride = stride
            return
        order = np.lexsort((post, pre))
        pre, post = pre[order], post[order]
        n_pre = self.src.num_neurons
        row_length = np.bincount(pre, minlength=n_pre).astype(np.uint32)
        stride = int(max(1, row_length.max(initial=0)))
        starts = np.concatenate(([0], np.cumsum(row_length)[:-1])).astype(np.int64)
        within = np.arange(len(pre), dtype=np.int64) - starts[pre]
        ind = np.zeros((n_pre, stride), dtype=np.uint32)
        ind[pre, within] = post
        self.set_ragged(row_length, ind)
        self._coo = (order, pre, within)

    def set_ragged(self, row_length, ind):
        """Adopt connectivity already in the reference's ragged layout."""
        ind = np.ascontiguousarray(ind, dtype=np.uint32)
        self.row_length_host = np.ascontiguousarray(row_length, dtype=np.uint32)
        self.ind_host = ind.reshape(self.src.num_neurons, -1)
        self.row_stride = self.ind_host.shape[1]

    def set_var_ragged(self, name, values):
        self.var_host[name] = np.ascontiguousarray(values)

    def set_var_coo(self, name, values):
        """Per-synapse values in the order the COO lists were given to set_sparse_connections."""
        order, pre, within = self._coo
        dtype = np.uint8 if name == "d" else np.float32
        out = np.zeros(self.ind_host.shape, dtype=dtype)
        out[pre, within] = np.asarray(values)[order]
        self.var_host[name] = out

    def pull_connectivity_from_device(self):
        """Host copies of rowLength / ind (needed after on-device connectivity initialisation)."""
        self.row_length_host = self.vars["rowLength"].pull_from_device().copy()
        self.ind_host = self.vars["ind"].pull_from_device().reshape(self.src.num_neurons, self.row_stride)

    def get_sparse_pre_inds(self):
        return np.repeat(np.arange(self.src.num_neurons, dtype=np.uint32), self.row_length_host)

    def get_sparse_post_inds(self):
        mask = np.arange(self.row_stride)[None, :] < self.row_length_host[:, None]
        return self.ind_host[mask]

    @property
    def pre_spike_event_recording_data(self):
        """[(times, ids)] per batch of the presynaptic spike-like events this projection is driven by
        (pygenn/genn_groups.py:397-406); needs spike_event_recording_enabled on the source population."""
        e = self.src.event_thresholds.index(float(self.wu.params["Epre"]))
        return self._model._decode_recording(self.src, f"recordSpkEvent{e}")

    @property
    def num_synapses(self):
        return int(self.row_length_host.sum())

    def get_var_values(self, name):
        """Pull a per-synapse variable and return the valid entries in row-major order."""
        a = self.vars[name].pull_from_device().reshape(self.src.num_neurons, self.row_stride)
        mask = np.arange(self.row_stride)[None, :] < self.row_length_host[:, None]
        return a[mask]


class GeNNModel:
    def __init__(self, precision="float", model_name="model", batch_size=1, dt=1.0, device=0):
        if precision != "float":
            raise NotImplementedError("only fp32 models are supported")
        self.name = model_name
        self.batch_size = int(batch_size)
        self.dt = float(dt)
        self.fuse_postsynaptic_models = False
        self.timing_enabled = False
        self._init_time = 0.0
        self._init_sparse_time = 0.0
        # validation mode: synaptic input is summed per postsynaptic neuron in the order of the reference's CPU backend
        # (no atomics; bit-identical accumulators, slow).  Read when the model is loaded.
        self.ordered_accumulation = False
        self.neuron_populations = {}
        self.synapse_populations = {}
        self.current_sources = {}
        self.timestep = 0
        self._runner = C.c_void_p()
        self._built = False
        self._loaded = False
        self._device = device
        self._arrays = []
        self.num_recording_timesteps = None
        self.seed = 0                       # seeds every on-device initialisation snippet (ModelSpec::setSeed)
        self._init_streams = 0              # one generator stream per array initialised on the device, in creation order

    # ------------------------------------------------------------------ description
    def add_neuron_population(self, pop_name, num_neurons, neuron, params=None, vars=None):
        if neuron not in ("LIF", "Izhikevich", "SpikeSourceArray"):
            raise NotImplementedError(f"neuron model {neuron}")
        if pop_name in self.neuron_populations:
            raise ValueError(f"duplicate neuron population {pop_name}")
        g = NeuronGroup(self, pop_name, num_neurons, neuron, params or {}, vars or {})
        self.neuron_populations[pop_name] = g
        return g

    def add_current_source(self, cs_name, current_source_model, pop, params=None, vars=None):
        if current_source_model not in ("DC", "ArrayNoise", "PoissonExp"):
            raise NotImplementedError(f"current source {current_source_model}")
        cs = CurrentSource(cs_name, current_source_model, pop, params or {})
        pop.current_sources.append(cs)
        self.current_sources[cs_name] = cs
        return cs

    def add_synapse_population(self, pop_name, matrix_type, source, target, weight_update_init, postsynaptic_init,
                               connectivity_init=None):
        if matrix_type not in ("SPARSE", "TOEPLITZ", "DENSE", "BITMASK", "PROCEDURAL"):
            raise NotImplementedError(f"matrix type {matrix_type}")
        if matrix_type == "PROCEDURAL":
            if connectivity_init is None or connectivity_init.snippet not in _abi.CONNECT_SNIPPETS:
                raise NotImplementedError("PROCEDURAL connectivity needs init_sparse_connectivity with FixedProbability, "
                                          "FixedProbabilityNoAutapse or FixedNumberPostWithReplacement")
            if weight_update_init.snippet not in ("StaticPulse", "StaticPulseConstantWeight"):
                raise NotImplementedError(f"PROCEDURAL connectivity with {weight_update_init.snippet}")
        if weight_update_init.snippet == "StaticPulseReverse" and (matrix_type != "SPARSE" or source.neuron == "SpikeSourceArray"):
            raise NotImplementedError("StaticPulseReverse needs SPARSE connectivity and a source population with an input current")
        if weight_update_init.snippet == "StaticGraded":
            if matrix_type != "SPARSE":
                raise NotImplementedError("StaticGraded needs SPARSE connectivity")
            if source.neuron == "SpikeSourceArray":
                raise ValueError("StaticGraded references the presynaptic variable V, which a spike source does not have")
        if matrix_type == "BITMASK" and weight_update_init.snippet != "StaticPulseConstantWeight":
            raise ValueError("BITMASK connectivity has no per-synapse variables: use StaticPulseConstantWeight")
        if matrix_type == "DENSE" and weight_update_init.snippet not in ("StaticPulse", "StaticPulseConstantWeight"):
            raise NotImplementedError(f"DENSE connectivity with {weight_update_init.snippet}")
        if matrix_type == "TOEPLITZ" and (connectivity_init is None or connectivity_init.snippet != "Conv2D"):
            raise ValueError("TOEPLITZ connectivity needs init_toeplitz_connectivity('Conv2D', ...)")
        s = SynapseGroup(self, pop_name, matrix_type, source, target, weight_update_init, postsynaptic_init, connectivity_init)
        self.synapse_populations[pop_name] = s
        source.out_syn.append(s)
        target.in_syn.append(s)
        return s

    # ------------------------------------------------------------------ build = finalise + derive constants
    def build(self):
        for n in self.neuron_populations.values():
            # fuse postsynaptic models (src/genn/genn/neuronGroup.cc:436): same snippet, same parameters,
            # same dendritic-delay depth, no state variables
            # fusing walks the incoming projections from the last one added to the first
            # (fuseSynapseGroups, src/genn/genn/neuronGroup.cc:41-96), which fixes both the child
            # order (it decides the order in which Isyn is summed) and the owner of a fused outPost
            n.fused_psm = []
            for s in reversed(n.in_syn):
                key = (s.ps.snippet, tuple(sorted(s.ps.params.items())), self._den_delay(s))
                target = None
                if self.fuse_postsynaptic_models:
                    for grp in n.fused_psm:
                        o = grp[0]
                        if (o.ps.snippet, tuple(sorted(o.ps.params.items())), self._den_delay(o)) == key:
                            target = grp
                            break
                if target is None:
                    n.fused_psm.append([s])
                    s.fused_ps_target = s
                else:
                    target.append(s)
                    s.fused_ps_target = target[0]
            if len(n.fused_psm) > _abi.MAX_PSM:
                raise NotImplementedError(f"{n.name}: more than {_abi.MAX_PSM} postsynaptic models after fusing")
            if len(n.current_sources) > _abi.MAX_CS:
                raise NotImplementedError(f"{n.name}: more than {_abi.MAX_CS} current sources")
            pre = [s for s in n.out_syn if s.wu.snippet == "STDPTrace"]
            post = [s for s in n.in_syn if s.wu.snippet == "STDPTrace"]
            if len(pre) > 1 or len(post) > 1:
                raise NotImplementedError(f"{n.name}: more than one plastic projection per side")
            # the built-in STDP (weightUpdateModels.h:345-367) keeps no traces: it reads both populations' spike times
            additive = [s for s in n.out_syn + n.in_syn if s.wu.snippet == "STDP"]
            n.num_delay_slots = max([s.axonal_delay_steps for s in n.out_syn], default=0) + 1
            # projections whose event condition and parameters agree share one queue (neuronGroup.cc:505-517)
            n.event_thresholds = []
            for s in n.out_syn:
                if s.wu.snippet == "StaticGraded" and float(s.wu.params["Epre"]) not in n.event_thresholds:
                    n.event_thresholds.append(float(s.wu.params["Epre"]))
            n.pre_output_syn = [s for s in n.out_syn if s.wu.snippet == "StaticPulseReverse"]
            if len(n.pre_output_syn) > _abi.MAX_PRE_OUTPUT:
                raise NotImplementedError(f"{n.name}: more than {_abi.MAX_PRE_OUTPUT} projections with presynaptic output")
            if len(n.event_thresholds) > _abi.MAX_SPK_EVENT:
                raise NotImplementedError(f"{n.name}: more than {_abi.MAX_SPK_EVENT} spike-like event conditions")
            n.pre_trace_owner = pre[0] if pre else None
            n.post_trace_owner = post[0] if post else None
            n.needs_spike_time = bool(pre or post or additive)
        self._built = True

    @staticmethod
    def _den_delay(s):
        return s.max_dendritic_delay_timesteps if s.wu.snippet == "StaticPulseDendriticDelay" else 0

    def _alloc(self, count, dtype, fill=None, device_only=False):
        a = Array(count, dtype, fill, device_only)
        self._arrays.append(a)
        return a

    def _alloc_device_init(self, count, dtype, init, stream=None):
        a = self._alloc(count, dtype, device_only=True)
        a.init_on_device(init, self.seed, self._next_stream() if stream is None else stream, self.dt)
        return a

    def _next_stream(self):
        self._init_streams += 1
        return self._init_streams

    # ------------------------------------------------------------------ load = allocate + push merged groups
    def load(self, num_recording_timesteps=None):
        if not self._built:
            raise RuntimeError("build() must be called before load()")
        lib = _abi.load()
        _abi.check(lib.gennmi_init(self._device))
        load_start = time.perf_counter()
        B = self.batch_size
        self.num_recording_timesteps = num_recording_timesteps
        dt32 = lit32(self.dt)
        _abi.check(lib.gennmi_runner_create(C.byref(self._runner), C.c_float(dt32), B))

        # ---- neuron-group arrays (runtime.cc:156-282)
        for n in self.neuron_populations.values():
            N = n.num_neurons
            if n.neuron == "SpikeSourceArray":
                for v in ("startSpike", "endSpike"):
                    a = self._alloc(B * N, np.uint32)
                    a.view[:] = np.broadcast_to(np.asarray(n.var_init[v], dtype=np.uint32), (B, N)).reshape(-1) \
                        if np.ndim(n.var_init[v]) < 2 else np.asarray(n.var_init[v], dtype=np.uint32).reshape(-1)
                    a.push_to_device()
                    n.vars[v] = a
                st = np.ascontiguousarray(n.extra_global_params["spikeTimes"], dtype=np.float32)
                a = self._alloc(max(1, st.size), np.float32)
                a.view[:st.size] = st
                a.push_to_device()
                n.vars["spikeTimes"] = a
            else:
                names = ("V", "RefracTime") if n.neuron == "LIF" else ("V", "U")
                for v in names:
                    if isinstance(n.var_init[v], VarInit):
                        n.vars[v] = self._alloc_device_init(B * N, np.float32, n.var_init[v])
                        continue
                    a = self._alloc(B * N, np.float32)
                    init = np.asarray(n.var_init[v], dtype=np.float32)
                    a.view[:] = np.broadcast_to(init, (B, N)).reshape(-1) if init.ndim < 2 else init.reshape(-1)
                    a.push_to_device()
                    n.vars[v] = a
            n.vars["spkCnt"] = self._alloc(B * n.num_delay_slots, np.uint32)
            n.vars["spk"] = self._alloc(B * n.num_delay_slots * N, np.uint32)
            for s in n.pre_output_syn:
                s.vars["outPre"] = self._alloc(B * N, np.float32)
            for e in range(len(n.event_thresholds)):
                n.vars[f"spkCntEvent{e}"] = self._alloc(B, np.uint32)
                n.vars[f"spkEvent{e}"] = self._alloc(B * N, np.uint32)
                if n.spike_event_recording_enabled:
                    if not num_recording_timesteps:
                        raise RuntimeError("Cannot use recording system without specifying number of recording timesteps")
                    n.vars[f"recordSpkEvent{e}"] = self._alloc(((N + 31) // 32) * B * num_recording_timesteps, np.uint32)
            if n.spike_recording_enabled:
                if not num_recording_timesteps:
                    raise RuntimeError("Cannot use recording system without specifying number of recording timesteps")
                n.vars["recordSpk"] = self._alloc(((N + 31) // 32) * B * num_recording_timesteps, np.uint32)
            if n.needs_spike_time:
                n.vars["sT"] = self._alloc(B * N, np.float32, fill=-FLT_MAX)      # -TIME_MAX, as the reference's initialize()
            for grp in n.fused_psm:
                owner = grp[0]
                owner.vars["outPost"] = self._alloc(B * N, np.float32)
                D = self._den_delay(owner)
                if D:
                    owner.vars["denDelay"] = self._alloc(B * D * N, np.float32)
                    owner.vars["denDelayPtr"] = self._alloc(1, np.uint32)
            if n.pre_trace_owner is not None:
                n.pre_trace_owner.vars["preTrace"] = self._alloc(B * N, np.float32, fill=n.pre_trace_owner.wu.pre_vars.get("preTrace", 0.0))
            if n.post_trace_owner is not None:
                n.post_trace_owner.vars["postTrace"] = self._alloc(B * N, np.float32, fill=n.post_trace_owner.wu.post_vars.get("postTrace", 0.0))
            for cs in n.current_sources:
                if cs.kind == "PoissonExp":
                    cs.vars["current"] = self._alloc(B * N, np.float32)
                    if cs.stream is None:
                        # by place in the name-ordered list of the model's current sources, as the backend adapter numbers them
                        cs.stream = 1000 + sorted(self.current_sources).index(cs.name)
                if cs.kind == "ArrayNoise":
                    noise = np.ascontiguousarray(cs.extra_global_params["noise"], dtype=np.float32)
                    if noise.size % N:
                        raise ValueError(f"{cs.name}: noise array is not a multiple of the population size")
                    a = self._alloc(noise.size, np.float32)
                    a.view[:] = noise.reshape(-1)
                    a.push_to_device()
                    cs.vars["noise"] = a

        # ---- synapse-group arrays (runtime.cc:330-402)
        for s in self.synapse_populations.values():
            if s.matrix_type == "SPARSE":
                n_pre = s.src.num_neurons
                if s.ind_host is None and s.conn is not None:
                    self._init_connectivity_on_device(s)
                elif s.ind_host is None:
                    raise RuntimeError(f"{s.name}: sparse connectivity has not been set")
                else:
                    for name, host, dtype in (("rowLength", s.row_length_host, np.uint32), ("ind", s.ind_host, np.uint32)):
                        a = self._alloc(host.size, dtype)
                        a.view[:] = host.reshape(-1)
                        a.push_to_device()
                        s.vars[name] = a
                if s.wu.snippet == "StaticPulseConstantWeight":
                    # the sparse kernels read a weight per synapse: the one weight is written out
                    s.vars["g"] = self._alloc(n_pre * s.row_stride, np.float32, fill=np.float32(lit32(s.wu.params["g"])))
                names = [] if s.wu.snippet == "StaticPulseConstantWeight" else ["g"] + (["d"] if s.wu.snippet == "StaticPulseDendriticDelay" else [])
                # weights a learning rule writes are READ_WRITE variables: one copy per batch (models.h VarAccess::READ_WRITE has
                # the batch dimension), every copy starting from the same initial values
                copies = B if s.wu.snippet in ("STDPTrace", "STDP") else 1
                for name in names:
                    dtype = np.uint8 if name == "d" else np.float32
                    if name in s.vars:          # (written together with the connectivity)
                        continue
                    if name not in s.var_host and isinstance(s.wu.vars[name], VarInit):
                        if copies != 1:
                            raise NotImplementedError(f"{s.name}: device-side initialisation of plastic weights with batch size > 1")
                        streams = getattr(s, "init_streams", None)
                        s.vars[name] = self._alloc_device_init(n_pre * s.row_stride, dtype, s.wu.vars[name], streams[1] if streams and name == "g" else None)
                        continue
                    a = self._alloc(copies * n_pre * s.row_stride, dtype)
                    if name in s.var_host:
                        a.view[:] = np.tile(np.asarray(s.var_host[name], dtype=dtype).reshape(-1), copies)
                    else:
                        a.view[:] = dtype(s.wu.vars[name])
                    a.push_to_device()
                    s.vars[name] = a
            elif s.matrix_type == "PROCEDURAL":
                # nothing is stored: the generator streams the stored matrix would have used are reserved in the same order
                s.row_stride = max_row_length(s.conn.snippet, s.conn.params, s.src.num_neurons, s.trg.num_neurons)
                if s.procedural_streams is None:        # (a caller that must reproduce another numbering sets them beforehand)
                    s.procedural_streams = [self._next_stream(), 0]
                    if s.wu.snippet == "StaticPulse" and isinstance(s.wu.vars["g"], VarInit):
                        s.procedural_streams[1] = self._next_stream()
            elif s.matrix_type == "DENSE":
                if s.wu.snippet == "StaticPulse":
                    count = s.src.num_neurons * s.trg.num_neurons
                    init = s.var_host.get("g", s.wu.vars.get("g"))
                    if isinstance(init, VarInit):
                        s.vars["g"] = self._alloc_device_init(count, np.float32, init)
                    else:
                        a = self._alloc(count, np.float32)
                        a.view[:] = np.broadcast_to(np.asarray(init, dtype=np.float32).reshape(-1), (count,)) if np.size(init) in (1, count) \
                            else np.asarray(init, dtype=np.float32).reshape(-1)
                        a.push_to_device()
                        s.vars["g"] = a
            elif s.matrix_type == "BITMASK":
                if s.gp_host is None:
                    raise RuntimeError(f"{s.name}: bitmask connectivity has not been set")
                a = self._alloc(s.gp_host.size, np.uint32)
                a.view[:] = s.gp_host
                a.push_to_device()
                s.vars["gp"] = a
            else:
                kern = np.ascontiguousarray(s.var_host.get("g", s.wu.vars.get("g")), dtype=np.float32)
                a = self._alloc(kern.size, np.float32)
                a.view[:] = kern.reshape(-1)
                a.push_to_device()
                s.vars["g"] = a

        _abi.check(lib.gennmi_synchronize())
        self._init_time += time.perf_counter() - load_start
        sparse_start = time.perf_counter()
        self._initialize_sparse()
        _abi.check(lib.gennmi_synchronize())
        self._init_sparse_time += time.perf_counter() - sparse_start
        self._push_merged_groups()
        if self.ordered_accumulation:
            _abi.check(lib.gennmi_runner_set_ordered(self._runner, 1))
        _abi.check(lib.gennmi_runner_finalise(self._runner))
        if self.timing_enabled:
            _abi.check(lib.gennmi_runner_set_timing(self._runner, 1))
        self._loaded = True
        self.timestep = 0

    def _init_connectivity_on_device(self, s):
        """Built-in connectivity snippets on the device (the reference's initializeSparse path for GPU backends)."""
        lib = _abi.load()
        n_pre, n_post = s.src.num_neurons, s.trg.num_neurons
        snippet, params = s.conn.snippet, s.conn.params
        multiple = getattr(s, "row_stride_multiple", 1)         # (the GeNN backend pads rows to 4 entries)
        s.row_stride = (max_row_length(snippet, params, n_pre, n_post) + multiple - 1) // multiple * multiple
        s.vars["rowLength"] = self._alloc(n_pre, np.uint32, device_only=True)
        s.vars["ind"] = self._alloc(n_pre * s.row_stride, np.uint32, device_only=True)
        row_length, ind = s.vars["rowLength"].ptr, s.vars["ind"].ptr
        # (a caller that must reproduce another numbering of the generator streams sets init_streams beforehand)
        stream = s.init_streams[0] if getattr(s, "init_streams", None) else self._next_stream()
        if snippet == "OneToOne":
            _abi.check(lib.gennmi_init_sparse_one_to_one(n_pre, n_post, s.row_stride, row_length, ind))
        elif snippet in ("FixedProbability", "FixedProbabilityNoAutapse"):
            _abi.check(lib.gennmi_init_sparse_fixed_probability(n_pre, n_post, s.row_stride, float(params["prob"]),
                                                                int(snippet.endswith("NoAutapse")), self.seed, stream, row_length, ind, None))
        elif snippet == "FixedNumberPostWithReplacement":
            _abi.check(lib.gennmi_init_sparse_fixed_number_post(n_pre, n_post, s.row_stride, int(params["num"]), None,
                                                                self.seed, stream, row_length, ind, None))
        elif snippet == "FixedNumberPreWithReplacement":
            _abi.check(lib.gennmi_init_sparse_fixed_number_pre(n_pre, n_post, s.row_stride, int(params["num"]),
                                                               self.seed, stream, row_length, ind, None))
        elif snippet == "Conv2D":
            conv = (C.c_int32 * 12)(*(int(params[k]) for k in _CONV2D_PARAMS))
            if conv[6] * conv[7] * conv[8] != n_pre or conv[9] * conv[10] * conv[11] != n_post:
                raise ValueError(f"{s.name}: Conv2D shapes do not match the populations' sizes")
            kernel = g = None
            init = s.wu.vars.get("g")
            if isinstance(init, VarInit) and init.snippet == "Kernel" and "g" not in s.var_host:
                values = np.ascontiguousarray(init.params["kernel"], dtype=np.float32).reshape(-1)
                if values.size != conv[0] * conv[1] * conv[8] * conv[11]:
                    raise ValueError(f"{s.name}: the kernel must hold conv_kh * conv_kw * conv_ic * conv_oc values")
                k = self._alloc(values.size, np.float32)
                k.view[:] = values
                k.push_to_device()
                s.vars["kernel"] = k
                s.vars["g"] = self._alloc(n_pre * s.row_stride, np.float32, device_only=True)
                kernel, g = k.ptr, s.vars["g"].ptr
            _abi.check(lib.gennmi_init_sparse_conv2d(conv, s.row_stride, row_length, ind, kernel, g, None))
        else:
            # FixedNumberTotalWithReplacement: the row lengths are one multinomial draw, made on the host as the
            # snippet's host init code does (initSparseConnectivitySnippet.h:312-358), then handed to the device
            rng = np.random.Generator(np.random.Philox(key=[self.seed, stream]))
            lengths = rng.multinomial(int(params["num"]), np.full(n_pre, 1.0 / n_pre)).astype(np.uint32)
            s.vars["rowLength"].view[:] = lengths
            s.vars["rowLength"].push_to_device()
            _abi.check(lib.gennmi_init_sparse_fixed_number_post(n_pre, n_post, s.row_stride, 0, row_length,
                                                                self.seed, stream, row_length, ind, None))

    def _initialize_sparse(self):
        """initializeSparse(): column views for projections with postsynaptic-spike code."""
        lib = _abi.load()
        for s in self.synapse_populations.values():
            if s.wu.snippet not in ("STDPTrace", "STDP"):
                continue
            n_pre, n_post = s.src.num_neurons, s.trg.num_neurons
            m = C.c_uint32()
            _abi.check(lib.gennmi_max_col_length(n_pre, n_post, s.row_stride, s.vars["rowLength"].ptr, s.vars["ind"].ptr, C.byref(m)))
            s.col_stride = max(1, int(m.value)) if not s.col_stride else s.col_stride
            s.vars["colLength"] = self._alloc(n_post, np.uint32)
            s.vars["remap"] = self._alloc(n_post * s.col_stride, np.uint32)
            _abi.check(lib.gennmi_build_remap(n_pre, n_post, s.row_stride, s.col_stride, s.vars["rowLength"].ptr,
                                              s.vars["ind"].ptr, s.vars["colLength"].ptr, s.vars["remap"].ptr))

    # merged-group membership as the reference would form it (same model code and structure)
    def _neuron_merge_key(self, n):
        psm = tuple((grp[0].ps.snippet, self._den_delay(grp[0])) for grp in self._sorted_psm(n))
        return (n.neuron, psm, tuple(cs.kind for cs in n.current_sources), n.pre_trace_owner is not None,
                n.post_trace_owner is not None, n.needs_spike_time, n.spike_recording_enabled, n.num_delay_slots, len(n.event_thresholds), len(n.pre_output_syn))

    def _sorted_psm(self, n):
        # children are ordered by a structure-only digest, ties keep creation order (groupMerged.h:411-454)
        return sorted(n.fused_psm, key=lambda grp: (grp[0].ps.snippet, self._den_delay(grp[0])))

    def _push_merged_groups(self):
        lib = _abi.load()
        B = self.batch_size
        merged = {}
        for n in self.neuron_populations.values():
            merged.setdefault(self._neuron_merge_key(n), []).append(n)
        for members in merged.values():
            model = members[0].neuron
            descs = [_abi.NeuronUpdateGroup() for _ in members]
            for d, n in zip(descs, members):
                d.model = {"LIF": _abi.NEURON_LIF, "Izhikevich": _abi.NEURON_IZHIKEVICH, "SpikeSourceArray": _abi.NEURON_SPIKE_SOURCE_ARRAY}[model]
                d.numNeurons = n.num_neurons
                d.spkCnt, d.spk = n.vars["spkCnt"].ptr, n.vars["spk"].ptr
                d.numDelaySlots = n.num_delay_slots
                d.recordSpk = n.vars["recordSpk"].ptr if "recordSpk" in n.vars else None
                d.sT = n.vars["sT"].ptr if "sT" in n.vars else None
            if model == "SpikeSourceArray":
                for d, n in zip(descs, members):
                    d.startSpike, d.endSpike, d.spikeTimes = n.vars["startSpike"].ptr, n.vars["endSpike"].ptr, n.vars["spikeTimes"].ptr
            elif model == "LIF":
                def derived(n):
                    p = n.params
                    return [p["Ioffset"], p["TauM"] / p["C"], p["Vrest"], math.exp(-self.dt / p["TauM"]), p["Vthresh"], p["Vreset"], p["TauRefrac"]]
                cols = list(zip(*[derived(n) for n in members]))
                rounded = [_merge_round(list(col)) for col in cols]
                for k, (d, n) in enumerate(zip(descs, members)):
                    d.var0, d.var1 = n.vars["V"].ptr, n.vars["RefracTime"].ptr
                    for j in range(7):
                        d.params[j] = rounded[j][k]
            else:
                cols = list(zip(*[[n.params[q] for q in ("a", "b", "c", "d")] for n in members]))
                rounded = [_merge_round(list(col)) for col in cols]
                for k, (d, n) in enumerate(zip(descs, members)):
                    d.var0, d.var1 = n.vars["V"].ptr, n.vars["U"].ptr
                    for j in range(4):
                        d.params[j] = rounded[j][k]
            for d, n in zip(descs, members):
                d.numPreOutput = len(n.pre_output_syn)
                for q, s in enumerate(n.pre_output_syn):
                    d.outPre[q] = s.vars["outPre"].ptr
            # spike-like event children
            for e in range(len(members[0].event_thresholds)):
                thresholds = _merge_round([n.event_thresholds[e] for n in members])
                for k, (d, n) in enumerate(zip(descs, members)):
                    d.numSpkEvent = len(n.event_thresholds)
                    d.spkEvent[e].spkCntEvent, d.spkEvent[e].spkEvent = n.vars[f"spkCntEvent{e}"].ptr, n.vars[f"spkEvent{e}"].ptr
                    d.spkEvent[e].threshold = thresholds[k]
                    if f"recordSpkEvent{e}" in n.vars:
                        d.spkEvent[e].recordSpkEvent = n.vars[f"recordSpkEvent{e}"].ptr
            # postsynaptic-model children
            num_psm = len(members[0].fused_psm)
            for m in range(num_psm):
                owners = [self._sorted_psm(n)[m][0] for n in members]
                if owners[0].ps.snippet == "ExpCurr":
                    taus = [o.ps.params["tau"] for o in owners]
                    decay = _merge_round([math.exp(-self.dt / tau) for tau in taus])
                    init = _merge_round([(tau * (1.0 - math.exp(-self.dt / tau))) * (1.0 / self.dt) for tau in taus])
                for k, (d, o) in enumerate(zip(descs, owners)):
                    p = d.psm[m]
                    p.outPost = o.vars["outPost"].ptr
                    D = self._den_delay(o)
                    p.maxDenDelay = D
                    if D:
                        p.denDelay, p.denDelayPtr = o.vars["denDelay"].ptr, o.vars["denDelayPtr"].ptr
                    if o.ps.snippet == "ExpCurr":
                        p.kind, p.init, p.expDecay = _abi.PSM_EXPCURR, init[k], decay[k]
                    else:
                        p.kind = _abi.PSM_DELTACURR
            for d in descs:
                d.numPSM = num_psm
            # current-source children
            num_cs = len(members[0].current_sources)
            for c in range(num_cs):
                srcs = [n.current_sources[c] for n in members]
                if srcs[0].kind == "DC":
                    amps = _merge_round([cs.params["amp"] for cs in srcs])
                if srcs[0].kind == "PoissonExp":
                    # the snippet's derived parameters (currentSourceModels.h:123-128)
                    dt = self.dt
                    decay = _merge_round([math.exp(-dt / cs.params["tauSyn"]) for cs in srcs])
                    init = _merge_round([cs.params["weight"] * (1.0 - math.exp(-dt / cs.params["tauSyn"])) * (cs.params["tauSyn"] / dt) for cs in srcs])
                    lam = _merge_round([math.exp(-(cs.params["rate"] / 1000.0) * dt) for cs in srcs])
                for k, (d, cs, n) in enumerate(zip(descs, srcs, members)):
                    if cs.kind == "PoissonExp":
                        d.cs[c].kind, d.cs[c].current = _abi.CS_POISSON_EXP, cs.vars["current"].ptr
                        d.cs[c].init, d.cs[c].expDecay, d.cs[c].expMinusLambda = init[k], decay[k], lam[k]
                        d.cs[c].seed, d.cs[c].stream = self.seed, cs.stream
                    elif cs.kind == "DC":
                        d.cs[c].kind, d.cs[c].amp = _abi.CS_DC, amps[k]
                    else:
                        d.cs[c].kind, d.cs[c].array = _abi.CS_ARRAY, cs.vars["noise"].ptr
                        d.cs[c].arraySteps = cs.vars["noise"].count // n.num_neurons
            for d in descs:
                d.numCS = num_cs
            # weight-update pre / post children (trace decay is a derived parameter of the WU model)
            if members[0].pre_trace_owner is not None:
                dec = _merge_round([math.exp(-self.dt / n.pre_trace_owner.wu.params["tauPlus"]) for n in members])
                for k, (d, n) in enumerate(zip(descs, members)):
                    d.preTrace, d.preDecay = n.pre_trace_owner.vars["preTrace"].ptr, dec[k]
            if members[0].post_trace_owner is not None:
                dec = _merge_round([math.exp(-self.dt / n.post_trace_owner.wu.params["tauMinus"]) for n in members])
                for k, (d, n) in enumerate(zip(descs, members)):
                    d.postTrace, d.postDecay = n.post_trace_owner.vars["postTrace"].ptr, dec[k]
            for d in descs:
                _abi.check(lib.gennmi_push_neuron_update_group(self._runner, C.byref(d), None))

        # presynaptic / postsynaptic update groups; merged by weight-update code and matrix type
        # (descriptors are pushed in the order the projections were added to the model, whatever their merged group: projections
        # that share a target are then added to it in that order under ordered accumulation, as the oracle's loop does)
        syn_merged = {}
        creation = {id(s): k for k, s in enumerate(self.synapse_populations.values())}
        pushes = []
        for s in self.synapse_populations.values():
            syn_merged.setdefault((s.matrix_type, s.wu.snippet, self._den_delay(s) > 0), []).append(s)
        for members in syn_merged.values():
            stdp = members[0].wu.snippet == "STDPTrace"
            additive = members[0].wu.snippet == "STDP"
            if stdp:
                rounded = {q: _merge_round([s.wu.params[q] for s in members]) for q in ("aPlus", "aMinus", "wMin", "wMax")}
            if additive:
                rounded = {q: _merge_round([s.wu.params[q] for s in members]) for q in ("tauPlus", "tauMinus", "Aplus", "Aminus", "Wmin", "Wmax")}
            if members[0].wu.snippet == "StaticPulseConstantWeight":
                consts = _merge_round([s.wu.params["g"] for s in members])
            if members[0].wu.snippet == "StaticGraded":
                graded = {q: _merge_round([s.wu.params[q] for s in members]) for q in ("Epre", "Vslope")}
            for k, s in enumerate(members):
                d = _abi.PresynapticUpdateGroup()
                d.matrix = {"SPARSE": _abi.MATRIX_SPARSE, "TOEPLITZ": _abi.MATRIX_TOEPLITZ_CONV2D, "DENSE": _abi.MATRIX_DENSE,
                            "BITMASK": _abi.MATRIX_BITMASK, "PROCEDURAL": _abi.MATRIX_PROCEDURAL}[s.matrix_type]
                d.wum = {"StaticPulse": _abi.WUM_STATIC_PULSE, "StaticPulseDendriticDelay": _abi.WUM_STATIC_PULSE_DENDRITIC_DELAY,
                         "STDPTrace": _abi.WUM_STDP_TRACE, "STDP": _abi.WUM_STDP, "StaticPulseConstantWeight": _abi.WUM_STATIC_PULSE_CONSTANT_WEIGHT,
                         "StaticGraded": _abi.WUM_STATIC_GRADED, "StaticPulseReverse": _abi.WUM_STATIC_PULSE_REVERSE}[s.wu.snippet]
                if s.wu.snippet == "StaticPulseConstantWeight":
                    d.constantWeight = consts[k]
                    if s.matrix_type == "SPARSE":
                        d.wum = _abi.WUM_STATIC_PULSE
                d.span = {"POSTSYNAPTIC": _abi.SPAN_AUTO, "PRESYNAPTIC": _abi.SPAN_PRE, "WAVE": _abi.SPAN_POST}[s.parallelism_hint]
                d.numThreadsPerSpike = s.num_threads_per_spike
                d.numSrcNeurons, d.numTrgNeurons = s.src.num_neurons, s.trg.num_neurons
                owner = s.fused_ps_target
                d.outPost = owner.vars["outPost"].ptr
                d.srcSpkCnt, d.srcSpk = s.src.vars["spkCnt"].ptr, s.src.vars["spk"].ptr
                d.axonalDelaySteps, d.numSrcDelaySlots = s.axonal_delay_steps, s.src.num_delay_slots
                if s.wu.snippet == "StaticPulseReverse":
                    d.outPre = s.vars["outPre"].ptr
                if s.wu.snippet == "StaticGraded":
                    # the projection is driven by the source's event queue for its threshold, not by its spikes
                    e = s.src.event_thresholds.index(float(s.wu.params["Epre"]))
                    d.srcSpkCnt, d.srcSpk = s.src.vars[f"spkCntEvent{e}"].ptr, s.src.vars[f"spkEvent{e}"].ptr
                    d.srcV = s.src.vars["V"].ptr
                    d.gradedEpre, d.gradedVslope = graded["Epre"][k], graded["Vslope"][k]
                if "g" in s.vars:
                    d.g = s.vars["g"].ptr
                if s.matrix_type == "BITMASK":
                    d.rowStride = s.row_stride
                    d.gp = s.vars["gp"].ptr
                if s.matrix_type == "PROCEDURAL":
                    d.rowStride = s.row_stride
                    q = d.procedural
                    q.seed = self.seed
                    q.connectivity = _abi.CONNECT_SNIPPETS[s.conn.snippet]
                    q.connectivityStream, q.weightStream = s.procedural_streams
                    q.prob = float(s.conn.params.get("prob", 0.0))
                    q.num = int(s.conn.params.get("num", 0))
                    if s.wu.snippet == "StaticPulse":
                        init = s.wu.vars["g"]
                        if isinstance(init, VarInit):
                            q.weightSnippet = _abi.INIT_SNIPPETS[init.snippet]
                            for j, v in enumerate(init.values(self.dt)):
                                q.weightParams[j] = v
                        else:
                            q.weightSnippet = _abi.INIT_SNIPPETS["Constant"]
                            q.weightParams[0] = float(init)
                if s.matrix_type in ("DENSE", "BITMASK", "PROCEDURAL"):
                    pass
                elif s.matrix_type == "SPARSE":
                    d.rowStride = s.row_stride
                    d.rowLength, d.ind = s.vars["rowLength"].ptr, s.vars["ind"].ptr
                    D = self._den_delay(s)
                    if D:
                        d.maxDenDelay = D
                        d.d = s.vars["d"].ptr
                        d.denDelay, d.denDelayPtr = owner.vars["denDelay"].ptr, owner.vars["denDelayPtr"].ptr
                else:
                    for j, q in enumerate(("conv_kh", "conv_kw", "conv_ih", "conv_iw", "conv_ic", "conv_oh", "conv_ow", "conv_oc")):
                        d.conv[j] = int(s.conn.params[q])
                if stdp:
                    d.trgST, d.postTrace = s.trg.vars["sT"].ptr, s.vars["postTrace"].ptr
                    d.aMinus, d.wMin, d.wMax = rounded["aMinus"][k], rounded["wMin"][k], rounded["wMax"][k]
                if additive:
                    d.trgST, d.tauMinus = s.trg.vars["sT"].ptr, rounded["tauMinus"][k]
                    d.aMinus, d.wMin, d.wMax = rounded["Aminus"][k], rounded["Wmin"][k], rounded["Wmax"][k]
                pushes.append((creation[id(s)], 0, d))
                if additive:
                    q = _abi.PostsynapticUpdateGroup()
                    q.numSrcNeurons, q.numTrgNeurons = s.src.num_neurons, s.trg.num_neurons
                    q.rowStride, q.colStride = s.row_stride, s.col_stride
                    q.colLength, q.remap, q.g = s.vars["colLength"].ptr, s.vars["remap"].ptr, s.vars["g"].ptr
                    q.trgSpkCnt, q.trgSpk = s.trg.vars["spkCnt"].ptr, s.trg.vars["spk"].ptr
                    q.srcST, q.tauPlus = s.src.vars["sT"].ptr, rounded["tauPlus"][k]
                    q.rowLength, q.ind = s.vars["rowLength"].ptr, s.vars["ind"].ptr
                    q.aPlus, q.wMin, q.wMax = rounded["Aplus"][k], rounded["Wmin"][k], rounded["Wmax"][k]
                    pushes.append((creation[id(s)], 1, q))
                if stdp:
                    q = _abi.PostsynapticUpdateGroup()
                    q.numSrcNeurons, q.numTrgNeurons = s.src.num_neurons, s.trg.num_neurons
                    q.rowStride, q.colStride = s.row_stride, s.col_stride
                    q.colLength, q.remap, q.g = s.vars["colLength"].ptr, s.vars["remap"].ptr, s.vars["g"].ptr
                    q.trgSpkCnt, q.trgSpk = s.trg.vars["spkCnt"].ptr, s.trg.vars["spk"].ptr
                    q.srcST, q.preTrace = s.src.vars["sT"].ptr, s.vars["preTrace"].ptr
                    q.rowLength, q.ind = s.vars["rowLength"].ptr, s.vars["ind"].ptr
                    q.aPlus, q.wMin, q.wMax = rounded["aPlus"][k], rounded["wMin"][k], rounded["wMax"][k]
                    pushes.append((creation[id(s)], 1, q))
        for _, post, desc in sorted(pushes, key=lambda e: (e[0], e[1])):
            if post:
                _abi.check(lib.gennmi_push_postsynaptic_update_group(self._runner, C.byref(desc), None))
            else:
                _abi.check(lib.gennmi_push_presynaptic_update_group(self._runner, C.byref(desc), None))

    # ------------------------------------------------------------------ stepping
    @property
    def t(self):
        return float(np.float32(self.timestep) * lit32(self.dt))

    def step_time(self):
        nrec = self.num_recording_timesteps or 0
        _abi.check(_abi.load().gennmi_step_time(self._runner, self.timestep, nrec))
        self.timestep += 1

    def update_synapses(self):
        """First half of step_time(): the runner's updateSynapses(t) on its own."""
        _abi.check(_abi.load().gennmi_update_synapses(self._runner, C.c_float(np.float32(self.timestep) * lit32(self.dt))))

    def update_neurons(self):
        """Second half of step_time(): the runner's updateNeurons(t, recordingTimestep); advances time."""
        nrec = self.num_recording_timesteps or 0
        _abi.check(_abi.load().gennmi_update_neurons(self._runner, C.c_float(np.float32(self.timestep) * lit32(self.dt)),
                                                     (self.timestep % nrec) if nrec else 0))
        self.timestep += 1

    def run(self, num_steps):
        """num_steps consecutive step_time() calls replayed from captured HIP graphs."""
        nrec = self.num_recording_timesteps or 0
        _abi.check(_abi.load().gennmi_run_steps(self._runner, self.timestep, int(num_steps), nrec))
        self.timestep += int(num_steps)

    def synchronize(self):
        _abi.check(_abi.load().gennmi_runner_synchronize(self._runner))

    def pull_recording_buffers_from_device(self):
        self.synchronize()
        for n in self.neuron_populations.values():
            for name, a in n.vars.items():
                if name.startswith("recordSpk"):
                    a.pull_from_device()

    def _decode_recording(self, n, var="recordSpk"):
        words = (n.num_neurons + 31) // 32
        rec = n.vars[var].view.reshape(self.num_recording_timesteps, self.batch_size, words)
        bits = np.unpackbits(rec.view(np.uint8), axis=2, bitorder="little")[:, :, :n.num_neurons]
        start = self.timestep - self.num_recording_timesteps if self.timestep >= self.num_recording_timesteps else 0
        out = []
        for b in range(self.batch_size):
            steps, ids = np.nonzero(bits[:, b, :])
            out.append(((start + steps).astype(np.float64) * self.dt, ids.astype(np.uint32)))
        return out

    @property
    def synaptic_event_count(self):
        v = C.c_ulonglong()
        _abi.check(_abi.load().gennmi_runner_event_count(self._runner, C.byref(v)))
        return int(v.value)

    def kernel_stats(self):
        st = (C.c_double * 8)()
        _abi.check(_abi.load().gennmi_runner_kernel_stats(self._runner, C.byref(st)))
        return {"presyn_launches": int(st[0]), "presyn_seconds": st[1], "neuron_launches": int(st[2]), "neuron_seconds": st[3],
                "postsyn_launches": int(st[4]), "postsyn_seconds": st[5], "step_launches": int(st[6]), "step_seconds": st[7]}

    def stream_mark(self, which):
        _abi.check(_abi.load().gennmi_runner_stream_mark(self._runner, int(which)))

    def stream_elapsed(self):
        v = C.c_double()
        _abi.check(_abi.load().gennmi_runner_stream_elapsed(self._runner, C.byref(v)))
        return v.value

    def runner_info(self):
        info = (C.c_uint32 * 4)()
        _abi.check(_abi.load().gennmi_runner_get_info(self._runner, C.byref(info)))
        return {"single_launch_step": bool(info[0] & 1), "resident_plan": bool(info[0] & 2), "bulk_neuron_kernel": bool(info[0] & 4), "ordered_accumulation": bool(info[0] & 8),
                "combined_synapse_launch": bool(info[0] & 16), "postsynaptic_in_combined_launch": bool(info[0] & 32),
                "conv_on_matrix_cores": bool(info[0] & 64), "conv_step_in_one_launch": bool(info[0] & 128), "neuron_blocks": info[1], "presyn_blocks": info[2], "postsyn_blocks": info[3]}

    # timing counters under PyGeNN's names (pygenn/genn_model.py:292-326), in seconds, accumulated while `timing_enabled`
    def _times(self):
        n, pre, post = C.c_double(), C.c_double(), C.c_double()
        _abi.check(_abi.load().gennmi_runner_get_times(self._runner, C.byref(n), C.byref(pre), C.byref(post)))
        return n.value, pre.value, post.value

    @property
    def neuron_update_time(self):
        return self._times()[0]

    @property
    def presynaptic_update_time(self):
        return self._times()[1]

    @property
    def postsynaptic_update_time(self):
        return self._times()[2]

    @property
    def init_time(self):
        """Wall-clock seconds load() spent allocating and initialising arrays (on the host or by the initialisation kernels)."""
        return self._init_time

    @property
    def init_sparse_time(self):
        """Wall-clock seconds load() spent on connectivity-dependent initialisation (column views of plastic projections)."""
        return self._init_sparse_time

    @property
    def synapse_dynamics_time(self):
        return 0.0          # no model of the supported set has synapse dynamics code

    def set_timing(self, enabled):
        _abi.check(_abi.load().gennmi_runner_set_timing(self._runner, int(bool(enabled))))

    def set_step_queue(self, max_steps):
        """Let step_time() leave up to max_steps steps queued in the library (a runner on the resident plan executes a
        queue in one launch); every pull, push, synchronisation and counter read executes the queue first.  0: off."""
        _abi.check(_abi.load().gennmi_runner_set_step_queue(self._runner, int(max_steps)))

    def unload(self):
        if self._runner:
            _abi.load().gennmi_runner_destroy(self._runner)
            self._runner = C.c_void_p()
        for a in self._arrays:
            a.free()
        self._arrays = []
        self._loaded = False


# --------------------------------------------------------------------------------------------
def model_from_net(net, batch_size=1, record=True, span=None, device=0, ordered=False):
    """Build a GeNNModel from a :class:`genn_amd.netspec.Net` (arrays are loaded, never generated here)."""
    m = GeNNModel("float", net.name, batch_size=batch_size, dt=net.dt, device=device)
    m.ordered_accumulation = bool(ordered)
    m.fuse_postsynaptic_models = net.fuse_psm
    pops = {}
    for p in net.pops:
        if p.model == "lif":
            g = m.add_neuron_population(p.name, p.n, "LIF", p.params, p.vars)
        elif p.model == "izh":
            g = m.add_neuron_population(p.name, p.n, "Izhikevich", p.params, p.vars)
        else:
            g = m.add_neuron_population(p.name, p.n, "SpikeSourceArray", {}, p.vars)
            g.set_extra_global_param("spikeTimes", p.spike_times)
        g.spike_recording_enabled = record
        pops[p.name] = g
    for c in net.css:
        if c.model == "poisson_exp":
            m.add_current_source(c.name, "PoissonExp", pops[c.pop], c.params)
        elif c.model == "dc":
            m.add_current_source(c.name, "DC", pops[c.pop], {"amp": c.amp})
        else:
            cs = m.add_current_source(c.name, "ArrayNoise", pops[c.pop])
            cs.set_extra_global_param("noise", c.noise)
    for s in net.syns:
        ps = init_postsynaptic("ExpCurr", {"tau": s.tau}) if s.psm == "expcurr" else init_postsynaptic("DeltaCurr")
        if s.wum == "static":
            wu = init_weight_update("StaticPulse", {}, {"g": 0.0})
        elif s.wum == "static_delay":
            wu = init_weight_update("StaticPulseDendriticDelay", {}, {"g": 0.0, "d": 0})
        elif s.wum == "static_const":
            wu = init_weight_update("StaticPulseConstantWeight", {"g": s.wum_params["g"]})
        elif s.wum == "static_graded":
            wu = init_weight_update("StaticGraded", s.wum_params, {"g": 0.0})
        elif s.wum == "static_reverse":
            wu = init_weight_update("StaticPulseReverse", {}, {"g": 0.0})
        else:
            wu = init_weight_update("STDPTrace", s.wum_params, {"g": 0.0}, {"preTrace": 0.0}, {"postTrace": 0.0})
        if s.wum == "stdp_additive":
            q = s.wum_params
            wu = init_weight_update("STDP", {"tauPlus": q["tauPlus"], "tauMinus": q["tauMinus"], "Aplus": q["aPlus"], "Aminus": q["aMinus"],
                                             "Wmin": q["wMin"], "Wmax": q["wMax"]}, {"g": 0.0})
        if s.matrix in ("procedural", "sparse_init"):
            if s.wum == "static":
                wu = init_weight_update("StaticPulse", {}, {"g": init_var(*s.g_init)})
            sg = m.add_synapse_population(s.name, "PROCEDURAL" if s.matrix == "procedural" else "SPARSE", pops[s.src], pops[s.trg], wu, ps,
                                          init_sparse_connectivity(*s.connect))
            # the numbering a GeNN model gets from the backend adapter: streams 2k + 1 and 2k + 2 for the k-th projection by name
            k = sorted(x.name for x in net.syns).index(s.name)
            if s.matrix == "procedural":
                sg.procedural_streams = [2 * k + 1, 2 * k + 2]
            else:
                sg.init_streams = [2 * k + 1, 2 * k + 2]
                sg.row_stride_multiple = 4
        elif s.matrix == "dense":
            sg = m.add_synapse_population(s.name, "DENSE", pops[s.src], pops[s.trg], wu, ps)
            if s.g is not None:
                sg.set_var_ragged("g", s.g)
        elif s.matrix == "bitmask":
            sg = m.add_synapse_population(s.name, "BITMASK", pops[s.src], pops[s.trg], wu, ps)
            sg.gp_host = np.ascontiguousarray(s.gp, dtype=np.uint32)
            sg.row_stride = s.row_stride
        elif s.matrix == "sparse":
            sg = m.add_synapse_population(s.name, "SPARSE", pops[s.src], pops[s.trg], wu, ps)
            sg.set_ragged(s.row_length, s.ind)
            if s.wum != "static_const":
                sg.set_var_ragged("g", s.g)
            if s.d is not None:
                sg.set_var_ragged("d", s.d)
            if s.max_den_delay:
                sg.max_dendritic_delay_timesteps = s.max_den_delay
            sg.axonal_delay_steps = s.axonal_delay_steps
            if s.hint_pre:
                sg.parallelism_hint = "PRESYNAPTIC"
                sg.num_threads_per_spike = s.threads_per_spike
            if span is not None:
                sg.parallelism_hint = span
        else:
            sg = m.add_synapse_population(s.name, "TOEPLITZ", pops[s.src], pops[s.trg], wu, ps,
                                          init_toeplitz_connectivity("Conv2D", s.conv))
            sg.set_var_ragged("g", s.g)
    m.seed = net.seed
    m.build()
    return m
