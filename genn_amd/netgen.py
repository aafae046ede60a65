"""ctypes binding of the multi-threaded synthetic-input generator (genn_amd/csrc/netgen.c).

Built in-tree by ``__graft_entry__.build()`` into genn_amd/lib/libgenn_netgen.so.  The streams are
the ones :mod:`genn_amd.rng` defines (tests check the two against each other word for word).
"""
import ctypes as C
import math
import os

import numpy as np

LIB_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "lib", "libgenn_netgen.so")
_lib = None

_u64, _u32, _f64, _vp = C.c_uint64, C.c_uint32, C.c_double, C.c_void_p


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(f"{LIB_PATH} is missing: run `python -c 'import __graft_entry__ as g; g.build()'` first")
        l = C.CDLL(LIB_PATH)
        l.ng_words.argtypes = [_u64, _u64, _u64, _u64, _vp]
        l.ng_uniform_f32.argtypes = [_u64, _u64, _u64, _u64, _f64, _f64, _vp]
        l.ng_normal_f32.argtypes = [_u64, _u64, _u64, _u64, _f64, _f64, _vp]
        l.ng_fixed_number_total_lengths.restype = _u32
        l.ng_fixed_number_total_lengths.argtypes = [_u64, _u64, _u32, _u64, _vp]
        l.ng_rows_uniform_targets.argtypes = [_u64, _u64, _u32, _u32, _vp, _u32, _vp]
        l.ng_fixed_probability.restype = _u32
        l.ng_fixed_probability.argtypes = [_u64, _u64, _u32, _u32, _f64, _u32, _vp, _u32, _vp]
        l.ng_rows_clipped_normal_f32.argtypes = [_u64, _u64, _u32, _vp, _u32, _f64, _f64, _f64, _f64, _vp]
        l.ng_rows_clipped_normal_delay_u8.argtypes = [_u64, _u64, _u32, _vp, _u32, _f64, _f64, _f64, _f64, _vp]
        l.ng_rows_uniform_f32.argtypes = [_u64, _u64, _u32, _vp, _u32, _u32, _f64, _f64, _f64, _f64, _vp]
        for name in ("ng_words", "ng_uniform_f32", "ng_normal_f32", "ng_rows_uniform_targets", "ng_rows_clipped_normal_f32",
                     "ng_rows_clipped_normal_delay_u8", "ng_rows_uniform_f32"):
            getattr(l, name).restype = None
        _lib = l
    return _lib


def _p(a):
    return a.ctypes.data_as(_vp)


def _pad(stride, pad):
    stride = max(1, int(stride))
    return ((stride + pad - 1) // pad) * pad


def words(seed, stream, start, count):
    out = np.empty(count, np.uint64)
    lib().ng_words(seed, stream, start, count, _p(out))
    return out


def uniform_f32(seed, stream, start, count, scale=1.0, offset=0.0):
    out = np.empty(count, np.float32)
    lib().ng_uniform_f32(seed, stream, start, count, scale, offset, _p(out))
    return out


def normal_f32(seed, stream, start, count, mean=0.0, sd=1.0):
    out = np.empty(count, np.float32)
    lib().ng_normal_f32(seed, stream, start, count, mean, sd, _p(out))
    return out


def fixed_number_total(seed, stream, n_pre, n_post, total, pad=1):
    """(rowLength, ind): `total` synapses, presynaptic and postsynaptic ends uniform with replacement."""
    row_length = np.empty(n_pre, np.uint32)
    longest = lib().ng_fixed_number_total_lengths(seed, stream, n_pre, total, _p(row_length))
    stride = _pad(longest, pad)
    ind = np.empty((n_pre, stride), np.uint32)
    lib().ng_rows_uniform_targets(seed, stream + 1, n_pre, n_post, _p(row_length), stride, _p(ind))
    return row_length, ind


def fixed_number_post(seed, stream, n_pre, n_post, fanout, pad=1):
    """(rowLength, ind): every row draws `fanout` targets uniformly with replacement, sorted."""
    row_length = np.full(n_pre, fanout, np.uint32)
    stride = _pad(fanout, pad)
    ind = np.empty((n_pre, stride), np.uint32)
    lib().ng_rows_uniform_targets(seed, stream, n_pre, n_post, _p(row_length), stride, _p(ind))
    return row_length, ind


def fixed_probability(seed, stream, n_pre, n_post, p, pad=1):
    """(rowLength, ind): Bernoulli(p) per (pre, post) pair."""
    mean = n_post * p
    budget = int(mean + 8.0 * math.sqrt(max(mean * (1 - p), 1.0)) + 16)
    row_length = np.empty(n_pre, np.uint32)
    longest = lib().ng_fixed_probability(seed, stream, n_pre, n_post, p, budget, _p(row_length), 0, None)
    if longest == 0xFFFFFFFF:
        raise RuntimeError("fixed_probability: counter budget exhausted")
    stride = _pad(longest, pad)
    ind = np.empty((n_pre, stride), np.uint32)
    lib().ng_fixed_probability(seed, stream, n_pre, n_post, p, budget, _p(row_length), stride, _p(ind))
    return row_length, ind


def rows_clipped_normal(seed, stream, row_length, stride, mean, sd, lo, hi):
    out = np.empty((len(row_length), stride), np.float32)
    lib().ng_rows_clipped_normal_f32(seed, stream, len(row_length), _p(row_length), stride, mean, sd, lo, hi, _p(out))
    return out


def rows_clipped_normal_delay(seed, stream, row_length, stride, mean, sd, lo, hi):
    out = np.empty((len(row_length), stride), np.uint8)
    lib().ng_rows_clipped_normal_delay_u8(seed, stream, len(row_length), _p(row_length), stride, mean, sd, lo, hi, _p(out))
    return out


def rows_uniform(seed, stream, row_length, stride, split, scale0, offset0, scale1, offset1):
    out = np.empty((len(row_length), stride), np.float32)
    lib().ng_rows_uniform_f32(seed, stream, len(row_length), _p(row_length), stride, split, scale0, offset0, scale1, offset1, _p(out))
    return out
