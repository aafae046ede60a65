"""ctypes binding of the C ABI declared in include/genn_mi355x.h (libgenn_mi355x.so).

The library is built in-tree by ``__graft_entry__.build()``; loading fails loudly when it is
missing — there is no CPU fallback anywhere in the package.
"""
import ctypes as C
import os

MAX_PSM = 8
MAX_CS = 4
MAX_EXTRA_SPK = 3
MAX_SPK_EVENT = 2
MAX_PRE_OUTPUT = 2

NEURON_LIF, NEURON_IZHIKEVICH, NEURON_SPIKE_SOURCE_ARRAY = 0, 1, 2
PSM_EXPCURR, PSM_DELTACURR = 0, 1
CS_DC, CS_ARRAY, CS_POISSON_EXP = 0, 1, 2
WUM_STATIC_PULSE, WUM_STATIC_PULSE_DENDRITIC_DELAY, WUM_STDP_TRACE, WUM_STATIC_PULSE_CONSTANT_WEIGHT, WUM_STATIC_GRADED, WUM_STATIC_PULSE_REVERSE, WUM_STDP = 0, 1, 2, 3, 4, 5, 6
MATRIX_SPARSE, MATRIX_TOEPLITZ_CONV2D, MATRIX_DENSE, MATRIX_BITMASK, MATRIX_PROCEDURAL = 0, 1, 2, 3, 4
CONNECT_SNIPPETS = {"FixedProbability": 0, "FixedProbabilityNoAutapse": 1, "FixedNumberPostWithReplacement": 2}
SPAN_AUTO, SPAN_POST, SPAN_PRE = 0, 1, 2

LIB_DIR = os.path.join(os.path.dirname(os.path.abspath(__file__)), "lib")
LIB_PATH = os.path.join(LIB_DIR, "libgenn_mi355x.so")

p_f32 = C.c_void_p
p_u32 = C.c_void_p
p_u8 = C.c_void_p


class Psm(C.Structure):
    _fields_ = [("outPost", p_f32), ("denDelay", p_f32), ("denDelayPtr", p_u32),
                ("init", C.c_float), ("expDecay", C.c_float), ("kind", C.c_uint32), ("maxDenDelay", C.c_uint32)]


class Cs(C.Structure):
    _fields_ = [("array", p_f32), ("amp", C.c_float), ("kind", C.c_uint32), ("arraySteps", C.c_uint32), ("stream", C.c_uint32),
                ("current", p_f32), ("init", C.c_float), ("expDecay", C.c_float), ("expMinusLambda", C.c_float), ("pad_", C.c_uint32),
                ("seed", C.c_uint64)]


class SpikeEvent(C.Structure):
    _fields_ = [("spkCntEvent", p_u32), ("spkEvent", p_u32), ("recordSpkEvent", p_u32), ("threshold", C.c_float), ("pad_", C.c_uint32)]


class NeuronUpdateGroup(C.Structure):
    _fields_ = [("model", C.c_uint32), ("numNeurons", C.c_uint32),
                ("var0", p_f32), ("var1", p_f32),
                ("startSpike", p_u32), ("endSpike", p_u32), ("spikeTimes", p_f32),
                ("params", C.c_float * 8),
                ("numPSM", C.c_uint32), ("numCS", C.c_uint32),
                ("psm", Psm * MAX_PSM), ("cs", Cs * MAX_CS),
                ("preTrace", p_f32), ("postTrace", p_f32),
                ("preDecay", C.c_float), ("postDecay", C.c_float),
                ("sT", p_f32), ("spkCnt", p_u32), ("spk", p_u32), ("recordSpk", p_u32),
                ("numExtraSpk", C.c_uint32), ("numDelaySlots", C.c_uint32),
                ("extraSpkCnt", p_u32 * MAX_EXTRA_SPK), ("extraSpk", p_u32 * MAX_EXTRA_SPK),
                ("numSpkEvent", C.c_uint32), ("numPreOutput", C.c_uint32), ("spkEvent", SpikeEvent * MAX_SPK_EVENT),
                ("outPre", p_f32 * MAX_PRE_OUTPUT)]


class Procedural(C.Structure):
    _fields_ = [("seed", C.c_uint64), ("connectivity", C.c_uint32), ("connectivityStream", C.c_uint32), ("prob", C.c_double),
                ("num", C.c_uint32), ("weightSnippet", C.c_uint32), ("weightStream", C.c_uint32), ("pad_", C.c_uint32),
                ("weightParams", C.c_double * 4)]


class PresynapticUpdateGroup(C.Structure):
    _fields_ = [("matrix", C.c_uint32), ("wum", C.c_uint32), ("span", C.c_uint32), ("numThreadsPerSpike", C.c_uint32),
                ("numSrcNeurons", C.c_uint32), ("numTrgNeurons", C.c_uint32),
                ("rowStride", C.c_uint32), ("maxDenDelay", C.c_uint32),
                ("rowLength", p_u32), ("ind", p_u32), ("g", p_f32), ("d", p_u8),
                ("outPost", p_f32), ("denDelay", p_f32), ("denDelayPtr", p_u32),
                ("srcSpkCnt", p_u32), ("srcSpk", p_u32),
                ("trgST", p_f32), ("postTrace", p_f32),
                ("aMinus", C.c_float), ("wMin", C.c_float), ("wMax", C.c_float),
                ("conv", C.c_int32 * 8),
                ("gp", p_u32), ("constantWeight", C.c_float), ("axonalDelaySteps", C.c_uint32),
                ("numSrcDelaySlots", C.c_uint32), ("tauMinus", C.c_float), ("procedural", Procedural),
                ("srcV", p_f32), ("gradedEpre", C.c_float), ("gradedVslope", C.c_float), ("outPre", p_f32)]


class PostsynapticUpdateGroup(C.Structure):
    _fields_ = [("numSrcNeurons", C.c_uint32), ("numTrgNeurons", C.c_uint32),
                ("rowStride", C.c_uint32), ("colStride", C.c_uint32),
                ("colLength", p_u32), ("remap", p_u32), ("g", p_f32),
                ("trgSpkCnt", p_u32), ("trgSpk", p_u32),
                ("srcST", p_f32), ("preTrace", p_f32),
                ("aPlus", C.c_float), ("wMin", C.c_float), ("wMax", C.c_float), ("tauPlus", C.c_float),
                ("rowLength", p_u32), ("ind", p_u32)]


INIT_SNIPPETS = {"Constant": 0, "Uniform": 1, "Normal": 2, "NormalClipped": 3, "NormalClippedDelay": 4, "Exponential": 5,
                 "Gamma": 6, "Binomial": 7}
ELEMENT_TYPES = {"float32": 0, "uint32": 1, "int32": 2, "uint16": 3, "uint8": 4}

# every symbol include/genn_mi355x.h declares: (restype, argtypes)
_ULL = C.c_ulonglong
SYMBOLS = {
    "gennmi_init": (C.c_int, [C.c_int]),
    "gennmi_last_error": (C.c_char_p, []),
    "gennmi_device_name": (C.c_int, [C.c_char_p, C.c_size_t]),
    "gennmi_malloc": (C.c_int, [C.POINTER(C.c_void_p), C.c_size_t]),
    "gennmi_free": (C.c_int, [C.c_void_p]),
    "gennmi_memcpy_to_device": (C.c_int, [C.c_void_p, C.c_void_p, C.c_size_t]),
    "gennmi_memcpy_from_device": (C.c_int, [C.c_void_p, C.c_void_p, C.c_size_t]),
    "gennmi_memset": (C.c_int, [C.c_void_p, C.c_int, C.c_size_t]),
    "gennmi_fill_f32": (C.c_int, [C.c_void_p, C.c_float, C.c_size_t]),
    "gennmi_copy_f32": (C.c_int, [C.c_void_p, C.c_void_p, C.c_size_t]),
    "gennmi_register_mirror": (C.c_int, [C.c_void_p, C.c_void_p, C.c_size_t]),
    "gennmi_unregister_mirror": (C.c_int, [C.c_void_p]),
    "gennmi_mirror_device_pointer": (C.c_int, [C.c_void_p, C.POINTER(C.c_void_p)]),
    "gennmi_push_mirrors": (C.c_int, []),
    "gennmi_register_device_array": (C.c_int, [C.c_void_p, C.c_void_p, C.c_size_t]),
    "gennmi_mirrors_begin_initialisation": (C.c_int, []),
    "gennmi_mirror_device_initialised": (C.c_int, [C.c_void_p]),
    "gennmi_mirror_ensure_host": (C.c_int, [C.c_void_p]),
    "gennmi_step": (C.c_int, [C.c_void_p, C.c_float, C.c_uint32]),
    "gennmi_synchronize": (C.c_int, []),
    "gennmi_note_device_write": (C.c_int, [C.c_void_p, C.c_size_t]),
    "gennmi_flush": (C.c_int, []),
    "gennmi_note_mirror_write": (C.c_int, [C.c_void_p]),
    "gennmi_free_device_memory_bytes": (C.c_int, [C.POINTER(C.c_size_t)]),
    "gennmi_abi_struct_sizes": (C.c_int, [C.POINTER(C.c_size_t * 5)]),
    "gennmi_runner_create": (C.c_int, [C.POINTER(C.c_void_p), C.c_float, C.c_uint32]),
    "gennmi_runner_destroy": (C.c_int, [C.c_void_p]),
    "gennmi_push_neuron_update_group": (C.c_int, [C.c_void_p, C.POINTER(NeuronUpdateGroup), C.POINTER(C.c_uint32)]),
    "gennmi_push_presynaptic_update_group": (C.c_int, [C.c_void_p, C.POINTER(PresynapticUpdateGroup), C.POINTER(C.c_uint32)]),
    "gennmi_push_postsynaptic_update_group": (C.c_int, [C.c_void_p, C.POINTER(PostsynapticUpdateGroup), C.POINTER(C.c_uint32)]),
    "gennmi_runner_finalise": (C.c_int, [C.c_void_p]),
    "gennmi_runner_set_ordered": (C.c_int, [C.c_void_p, C.c_int]),
    "gennmi_runner_set_step_queue": (C.c_int, [C.c_void_p, C.c_uint32]),
    "gennmi_build_remap": (C.c_int, [C.c_uint32, C.c_uint32, C.c_uint32, C.c_uint32, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p]),
    "gennmi_max_col_length": (C.c_int, [C.c_uint32, C.c_uint32, C.c_uint32, C.c_void_p, C.c_void_p, C.POINTER(C.c_uint32)]),
    "gennmi_max_col_length_static": (C.c_int, [C.c_uint32, C.c_uint32, C.c_uint32, C.c_void_p, C.c_void_p, C.c_void_p]),
    # generated code objects behind the C ABI (bound by generated C++ host code; listed so that the table and the header agree)
    "gennmi_program_create": (C.c_int, [C.POINTER(C.c_void_p), C.c_void_p, C.c_uint32]),
    "gennmi_program_destroy": (C.c_int, [C.c_void_p]),
    "gennmi_program_load_module": (C.c_int, [C.c_void_p, C.c_void_p, C.c_size_t, C.POINTER(C.c_uint32)]),
    "gennmi_program_get_kernel": (C.c_int, [C.c_void_p, C.c_uint32, C.c_char_p, C.POINTER(C.c_uint32)]),
    "gennmi_program_error_flag": (C.c_int, [C.c_void_p, C.POINTER(C.c_void_p)]),
    "gennmi_program_add_launch": (C.c_int, [C.c_void_p, C.c_int, C.c_uint32, C.c_uint32, C.c_uint32, C.c_uint32, C.c_void_p, C.c_size_t, C.c_int]),
    "gennmi_program_clear_phases": (C.c_int, [C.c_void_p]),
    "gennmi_program_update": (C.c_int, [C.c_void_p, C.c_int, C.c_double, C.c_uint32]),
    "gennmi_program_launch": (C.c_int, [C.c_void_p, C.c_uint32, C.c_uint32, C.c_uint32, C.c_uint32, C.c_void_p, C.c_size_t, C.c_double,
                                        C.c_ulonglong, C.c_int]),
    "gennmi_program_synchronize": (C.c_int, [C.c_void_p]),
    "gennmi_program_set_timing": (C.c_int, [C.c_void_p, C.c_int]),
    "gennmi_program_get_time": (C.c_int, [C.c_void_p, C.c_int, C.POINTER(C.c_double)]),
    "gennmi_program_get_info": (C.c_int, [C.c_void_p, C.POINTER(C.c_ulonglong * 4)]),
    "gennmi_host_malloc": (C.c_int, [C.POINTER(C.c_void_p), C.c_size_t, C.c_int, C.POINTER(C.c_void_p)]),
    "gennmi_host_free": (C.c_int, [C.c_void_p]),
    "gennmi_profiler_range_push": (C.c_int, [C.c_char_p]),
    "gennmi_profiler_range_pop": (C.c_int, []),
    "gennmi_init_var": (C.c_int, [C.c_void_p, C.c_uint32, C.c_size_t, C.c_uint32, C.POINTER(C.c_double * 4), C.c_uint64, C.c_uint32]),
    "gennmi_init_sparse_fixed_probability": (C.c_int, [C.c_uint32, C.c_uint32, C.c_uint32, C.c_double, C.c_int, C.c_uint64, C.c_uint32,
                                                       C.c_void_p, C.c_void_p, C.POINTER(C.c_uint32)]),
    "gennmi_init_sparse_fixed_number_post": (C.c_int, [C.c_uint32, C.c_uint32, C.c_uint32, C.c_uint32, C.c_void_p, C.c_uint64, C.c_uint32,
                                                       C.c_void_p, C.c_void_p, C.POINTER(C.c_uint32)]),
    "gennmi_init_sparse_fixed_number_pre": (C.c_int, [C.c_uint32, C.c_uint32, C.c_uint32, C.c_uint32, C.c_uint64, C.c_uint32,
                                                      C.c_void_p, C.c_void_p, C.POINTER(C.c_uint32)]),
    "gennmi_init_sparse_conv2d": (C.c_int, [C.POINTER(C.c_int32), C.c_uint32, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p,
                                            C.POINTER(C.c_uint32)]),
    "gennmi_init_sparse_one_to_one": (C.c_int, [C.c_uint32, C.c_uint32, C.c_uint32, C.c_void_p, C.c_void_p]),
    "gennmi_philox4x32": (C.c_int, [C.POINTER(C.c_uint32 * 4), C.POINTER(C.c_uint32 * 2), C.POINTER(C.c_uint32 * 4)]),
    "gennmi_init_random_words": (C.c_int, [C.c_void_p, C.c_size_t, C.c_uint64, C.c_uint32]),
    "gennmi_update_synapses": (C.c_int, [C.c_void_p, C.c_float]),
    "gennmi_update_neurons": (C.c_int, [C.c_void_p, C.c_float, C.c_uint32]),
    "gennmi_step_time": (C.c_int, [C.c_void_p, _ULL, _ULL]),
    "gennmi_run_steps": (C.c_int, [C.c_void_p, _ULL, _ULL, _ULL]),
    "gennmi_runner_synchronize": (C.c_int, [C.c_void_p]),
    "gennmi_runner_set_timing": (C.c_int, [C.c_void_p, C.c_int]),
    "gennmi_runner_get_times": (C.c_int, [C.c_void_p, C.POINTER(C.c_double), C.POINTER(C.c_double), C.POINTER(C.c_double)]),
    "gennmi_runner_kernel_stats": (C.c_int, [C.c_void_p, C.POINTER(C.c_double * 8)]),
    "gennmi_runner_stream_mark": (C.c_int, [C.c_void_p, C.c_int]),
    "gennmi_runner_stream_elapsed": (C.c_int, [C.c_void_p, C.POINTER(C.c_double)]),
    "gennmi_runner_get_info": (C.c_int, [C.c_void_p, C.POINTER(C.c_uint32 * 4)]),
    "gennmi_runner_event_count": (C.c_int, [C.c_void_p, C.POINTER(_ULL)]),
}

_lib = None


class GennmiError(RuntimeError):
    """Raised for any non-zero return of the C ABI (the reference throws std::runtime_error)."""


def load():
    """Load libgenn_mi355x.so and declare every prototype.  Raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise GennmiError(f"{LIB_PATH} is missing: run `python -c 'import __graft_entry__ as g; g.build()'` first")
        lib = C.CDLL(LIB_PATH, mode=C.RTLD_GLOBAL)
        for name, (res, args) in SYMBOLS.items():
            fn = getattr(lib, name)
            fn.restype = res
            fn.argtypes = args
        _lib = lib
    return _lib


def check(rc):
    if rc != 0:
        raise GennmiError(f"genn_mi355x error {rc}: {load().gennmi_last_error().decode()}")
