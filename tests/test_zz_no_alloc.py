"""The entry point that allocates nothing (gennmi_max_col_length_static) against the allocating one it is a variant of
(gennmi_max_col_length): same connectivity, bit-equal result — on two calls in a row, the second on a smaller matrix, so
that counters left behind by the first call would show."""
import ctypes as C

import numpy as np
import pytest

from genn_amd import _abi, netgen

pytestmark = pytest.mark.gpu


def _upload(lib, a):
    p = C.c_void_p()
    _abi.check(lib.gennmi_malloc(C.byref(p), a.nbytes))
    _abi.check(lib.gennmi_memcpy_to_device(p, a.ctypes.data_as(C.c_void_p), a.nbytes))
    return p


def test_static_max_col_length_matches_allocating_entry_point():
    lib = _abi.load()
    _abi.check(lib.gennmi_init(0))
    result_dev = C.c_void_p()
    _abi.check(lib.gennmi_malloc(C.byref(result_dev), 4))
    cases = ((6000, 5000, 0.05, 41), (1500, 700, 0.1, 42))       # the second has fewer rows and fewer columns
    for num_src, num_trg, prob, stream in cases:
        row_length, ind = netgen.fixed_probability(1234, stream, num_src, num_trg, prob)
        stride = ind.shape[1]
        d_rl, d_ind = _upload(lib, row_length), _upload(lib, np.ascontiguousarray(ind))
        want = C.c_uint32()
        _abi.check(lib.gennmi_max_col_length(num_src, num_trg, stride, d_rl, d_ind, C.byref(want)))
        _abi.check(lib.gennmi_max_col_length_static(num_src, num_trg, stride, d_rl, d_ind, result_dev))
        got = np.zeros(1, np.uint32)
        _abi.check(lib.gennmi_memcpy_from_device(got.ctypes.data_as(C.c_void_p), result_dev, 4))
        # independent of both: in-degrees counted on the host
        valid = np.arange(stride)[None, :] < row_length[:, None]
        host = int(np.bincount(ind[valid], minlength=num_trg).max())
        assert int(got[0]) == int(want.value) == host, (num_src, num_trg, int(got[0]), int(want.value), host)
        _abi.check(lib.gennmi_free(d_rl))
        _abi.check(lib.gennmi_free(d_ind))
    _abi.check(lib.gennmi_free(result_dev))


def test_static_max_col_length_rejects_sizes_beyond_its_array():
    lib = _abi.load()
    _abi.check(lib.gennmi_init(0))
    dummy = C.c_void_p()
    _abi.check(lib.gennmi_malloc(C.byref(dummy), 64))
    rc = lib.gennmi_max_col_length_static(1, (1 << 20) + 1, 4, dummy, dummy, dummy)
    assert rc == -2 and b"exceed" in lib.gennmi_last_error()
    _abi.check(lib.gennmi_free(dummy))
