"""On-device initialisation snippets, tested the way the reference tests its own (tests/features/test_connect_init.py,
tests/features/test_rng.py::test_init): exact structural invariants, and distributions by chi-square / Kolmogorov-Smirnov
at the reference's significance levels.  Everything here is seeded, so a pass or a fail is reproducible.

The generator under the snippets is pinned exactly: Philox4x32-10 against the known-answer vectors of its authors and
against an independent numpy restatement (tests/test_host_cpu.py holds the same check for the host entry point).
"""
import ctypes as C

import numpy as np
import pytest
from scipy import stats

from genn_amd import _abi
from genn_amd.genn_model import (GeNNModel, init_postsynaptic, init_sparse_connectivity, init_var, init_weight_update,
                                 max_row_length)
from philox_ref import philox4x32

pytestmark = pytest.mark.gpu

# significance levels of the reference's tests (test_connect_init.py:56-66, test_rng.py:168-176)
P_CONNECT = 0.0020
P_VAR = 0.00034


def _device_array(count, dtype):
    from genn_amd.genn_model import Array
    return Array(count, dtype, device_only=True)


def _init(count, dtype, snippet, params, seed=1234, stream=1):
    lib = _abi.load()
    _abi.check(lib.gennmi_init(0))
    a = _device_array(count, dtype)
    p = (C.c_double * 4)(*(list(params) + [0.0] * (4 - len(params))))
    _abi.check(lib.gennmi_init_var(a.ptr, _abi.ELEMENT_TYPES[np.dtype(dtype).name], count, _abi.INIT_SNIPPETS[snippet], C.byref(p), seed, stream))
    out = a.pull_from_device().copy()
    a.free()
    return out


def test_device_words_are_philox4x32_10():
    lib = _abi.load()
    _abi.check(lib.gennmi_init(0))
    count, seed, stream = 4099, 0x0123456789ABCDEF, 77
    a = _device_array(count, np.uint32)
    _abi.check(lib.gennmi_init_random_words(a.ptr, count, seed, stream))
    got = a.pull_from_device().copy()
    a.free()
    groups = np.arange((count + 3) // 4, dtype=np.uint64)
    want = philox4x32(groups & np.uint64(0xFFFFFFFF), groups >> np.uint64(32), 0, stream, seed & 0xFFFFFFFF, seed >> 32)
    assert np.array_equal(got, np.stack(want, axis=1).reshape(-1)[:count])


@pytest.mark.parametrize("count", [1, 3, 4, 1001, 1 << 20])
def test_var_init_is_a_function_of_seed_and_stream_only(count):
    a = _init(count, np.float32, "Uniform", [0.0, 1.0], seed=5, stream=9)
    b = _init(count, np.float32, "Uniform", [0.0, 1.0], seed=5, stream=9)
    c = _init(count, np.float32, "Uniform", [0.0, 1.0], seed=5, stream=10)
    d = _init(count, np.float32, "Uniform", [0.0, 1.0], seed=6, stream=9)
    assert np.array_equal(a, b)
    if count > 3:
        assert not np.array_equal(a, c) and not np.array_equal(a, d)
    # a longer array starts with the shorter one: element i never depends on the array length or the launch geometry
    longer = _init(count + 13, np.float32, "Uniform", [0.0, 1.0], seed=5, stream=9)
    assert np.array_equal(longer[:count], a)


def test_var_init_distributions():
    n = 50000           # population size of the reference's test_init
    cases = [("Uniform", [0.0, 1.0], stats.uniform.cdf, ()),
             ("Uniform", [-3.0, 5.0], stats.uniform(-3.0, 8.0).cdf, ()),
             ("Normal", [0.0, 1.0], stats.norm.cdf, ()),
             ("Normal", [-58.0, 5.0], stats.norm(-58.0, 5.0).cdf, ()),
             ("Exponential", [1.0], stats.expon.cdf, ()),
             ("Exponential", [2.5], stats.expon(scale=2.5).cdf, ()),          # value = lambda * Exp(1), initVarSnippet.h:223
             ("Gamma", [4.0, 1.0], stats.gamma.cdf, (4.0,)),
             ("Gamma", [0.5, 2.0], stats.gamma(0.5, scale=2.0).cdf, ()),
             ("NormalClipped", [1.0, 2.0, 0.0, 3.0], stats.truncnorm(-0.5, 1.0, loc=1.0, scale=2.0).cdf, ())]
    for stream, (snippet, params, cdf, args) in enumerate(cases, start=1):
        v = _init(n, np.float32, snippet, params, stream=stream)
        assert np.isfinite(v).all()
        p = stats.kstest(v.astype(np.float64), cdf, args).pvalue
        assert p > P_VAR, f"{snippet}{params} fails the KS test (p={p})"
    v = _init(n, np.float32, "NormalClipped", [1.0, 2.0, 0.0, 3.0], stream=20)
    assert v.min() >= 0.0 and v.max() <= 3.0
    assert np.all(_init(1000, np.float32, "Constant", [0.25]) == np.float32(0.25))


def test_var_init_binomial():
    for stream, (trials, prob) in enumerate([(20, 0.5), (1000, 0.01), (5000, 0.9), (7, 0.0), (7, 1.0)], start=1):
        v = _init(50000, np.uint32, "Binomial", [trials, prob], stream=stream)
        assert v.max() <= trials
        if prob in (0.0, 1.0):
            assert np.all(v == trials * prob)
            continue
        lo, hi = int(stats.binom.ppf(1e-4, trials, prob)), int(stats.binom.ppf(1.0 - 1e-4, trials, prob))
        obs = np.bincount(np.clip(v, lo, hi), minlength=hi + 1)[lo:hi + 1].astype(np.float64)
        cdf = stats.binom.cdf(np.arange(lo, hi + 1), trials, prob)
        exp = np.diff(np.concatenate(([0.0], cdf[:-1], [1.0]))) * len(v)            # tails folded into the end bins
        p = stats.chisquare(obs, exp).pvalue
        assert p > P_VAR, f"Binomial({trials}, {prob}) fails the chi-square test (p={p})"


def test_var_init_delay_is_integral_and_clipped():
    # NormalClippedDelay as the cortical microcircuit uses it: mean 1.5 ms, sd 0.75 ms, [0, 4.2] ms at dt = 0.1 ms
    dt = 0.1
    params = [1.5 / dt, 0.75 / dt, 0.0, 4.2 / dt]
    for dtype in (np.uint8, np.float32):
        v = _init(200003, dtype, "NormalClippedDelay", params, stream=3)
        assert v.min() >= 0 and v.max() <= 42
        assert np.all(v == np.rint(v))
        # rint of a clipped normal: compare the integer histogram with the truncated normal's mass per rounding interval
        tn = stats.truncnorm((0.0 - params[0]) / params[1], (params[3] - params[0]) / params[1], loc=params[0], scale=params[1])
        edges = np.concatenate(([0.0], np.arange(0.5, 42.0, 1.0), [42.0]))
        exp = np.diff(tn.cdf(edges)) * len(v)
        obs = np.bincount(v.astype(np.int64), minlength=43).astype(np.float64)
        p = stats.chisquare(obs, exp).pvalue
        assert p > P_VAR, f"{np.dtype(dtype).name}: NormalClippedDelay fails the chi-square test (p={p})"


_LIF = {"C": 1.0, "TauM": 20.0, "Vrest": -60.0, "Vreset": -60.0, "Vthresh": -50.0, "Ioffset": 0.0, "TauRefrac": 5.0}


def _empty_model(seed=0):
    m = GeNNModel("float", "init", dt=1.0)
    m.seed = seed
    return m


def _static(g=1.0):
    return init_weight_update("StaticPulse", {}, {"g": g})


def test_connect_init():
    """tests/features/test_connect_init.py with its sizes and checks, plus ordering and range."""
    model = _empty_model(seed=42)
    pre = model.add_neuron_population("Pre", 100, "LIF", _LIF, {"V": 0.0, "RefracTime": 0.0})
    post = model.add_neuron_population("Post", 100, "LIF", _LIF, {"V": 0.0, "RefracTime": 0.0})
    total = model.add_synapse_population("FixedNumberTotal", "SPARSE", pre, post, _static(), init_postsynaptic("DeltaCurr"),
                                         init_sparse_connectivity("FixedNumberTotalWithReplacement", {"num": 1000}))
    fixed_post = model.add_synapse_population("FixedNumberPost", "SPARSE", pre, post, _static(), init_postsynaptic("DeltaCurr"),
                                              init_sparse_connectivity("FixedNumberPostWithReplacement", {"num": 10}))
    fixed_pre = model.add_synapse_population("FixedNumberPre", "SPARSE", pre, post, _static(), init_postsynaptic("DeltaCurr"),
                                             init_sparse_connectivity("FixedNumberPreWithReplacement", {"num": 10}))
    one = model.add_synapse_population("OneToOne", "SPARSE", pre, post, _static(), init_postsynaptic("DeltaCurr"),
                                       init_sparse_connectivity("OneToOne"))
    model.build()
    model.load()
    for s in (total, fixed_post, fixed_pre, one):
        s.pull_connectivity_from_device()
        assert s.get_sparse_post_inds().max() < 100
        for r in range(100):
            row = s.ind_host[r, :s.row_length_host[r]]
            assert np.all(np.diff(row.astype(np.int64)) >= 0), f"{s.name}: row {r} is not ascending"
    assert np.all(np.bincount(fixed_post.get_sparse_pre_inds()) == 10)
    assert np.all(np.bincount(fixed_pre.get_sparse_post_inds()) == 10)
    assert stats.chisquare(np.bincount(fixed_pre.get_sparse_pre_inds(), minlength=100)).pvalue > P_CONNECT
    assert len(total.get_sparse_pre_inds()) == 1000
    assert np.array_equal(one.get_sparse_pre_inds(), one.get_sparse_post_inds())
    assert stats.chisquare(np.bincount(fixed_post.get_sparse_post_inds(), minlength=100)).pvalue > P_CONNECT
    assert stats.chisquare(np.bincount(total.get_sparse_post_inds(), minlength=100)).pvalue > P_CONNECT
    assert stats.chisquare(np.bincount(total.get_sparse_pre_inds(), minlength=100)).pvalue > P_CONNECT
    model.unload()


def _connectivity(snippet, params, num_pre, num_post, seed=7):
    model = _empty_model(seed)
    pre = model.add_neuron_population("Pre", num_pre, "LIF", _LIF, {"V": 0.0, "RefracTime": 0.0})
    post = model.add_neuron_population("Post", num_post, "LIF", _LIF, {"V": 0.0, "RefracTime": 0.0})
    s = model.add_synapse_population("S", "SPARSE", pre, post, _static(), init_postsynaptic("DeltaCurr"),
                                     init_sparse_connectivity(snippet, params))
    model.build()
    model.load()
    s.pull_connectivity_from_device()
    row_length, ind = s.row_length_host.copy(), s.ind_host.copy()
    model.unload()
    return row_length, ind


def test_fixed_number_post_rows_are_sorted_uniform_samples():
    """A row of FixedNumberPostWithReplacement must be the order statistics of `num` independent uniform targets
    (initSparseConnectivitySnippet.h:233-253).  Pinned against what the mathematics fixes: the k-th smallest of n uniforms
    is Beta(k, n+1-k); a dropped tail spacing would pin the largest target to the last neuron, a wrong normalisation would
    shift every mean k/(n+1)."""
    n, rows, num_post = 10, 20000, 1 << 20
    row_length, ind = _connectivity("FixedNumberPostWithReplacement", {"num": n}, rows, num_post)
    assert np.all(row_length == n)
    assert np.all(np.diff(ind.astype(np.int64), axis=1) >= 0)
    x = (ind.astype(np.float64) + 0.5) / num_post
    for k in (1, 2, 5, 9, 10):
        p = stats.kstest(x[:, k - 1], stats.beta(k, n + 1 - k).cdf).pvalue
        assert p > P_CONNECT, f"order statistic {k} of {n} fails the KS test (p={p})"
    # all targets pooled are uniform, and different rows are different
    assert stats.kstest(x.reshape(-1), stats.uniform.cdf).pvalue > P_CONNECT
    assert len(np.unique(ind, axis=0)) == rows


def test_fixed_number_post_long_rows():
    """Rows longer than a wavefront (several scan rounds) and not a multiple of 64."""
    n, rows, num_post = 1000, 512, 100000
    row_length, ind = _connectivity("FixedNumberPostWithReplacement", {"num": n}, rows, num_post)
    assert np.all(row_length == n) and ind.shape == (rows, n)
    assert np.all(np.diff(ind.astype(np.int64), axis=1) >= 0) and ind.max() < num_post
    x = (ind.astype(np.float64) + 0.5) / num_post
    for k in (1, 64, 65, 500, 1000):
        p = stats.kstest(x[:, k - 1], stats.beta(k, n + 1 - k).cdf).pvalue
        assert p > P_CONNECT, f"order statistic {k} of {n} fails the KS test (p={p})"
    assert stats.chisquare(np.bincount(ind.reshape(-1) // 1000, minlength=100)).pvalue > P_CONNECT


@pytest.mark.parametrize("num_pre,num_post,num", [(1000, 20000, 50), (37, 5000, 3), (20000, 300, 1000), (1, 100, 7), (3, 1500, 30)])
def test_fixed_number_pre(num_pre, num_post, num):
    """FixedNumberPreWithReplacement (initSparseConnectivitySnippet.h:380-410): every column holds exactly `num` entries
    (tests/features/test_connect_init.py:55), the sources of one column are independent uniform draws (so the pooled
    sources are uniform, row lengths are Binomial(num * numPost, 1 / numPre) and the number of DISTINCT sources of a column
    follows the occupancy law), rows come out ascending and nothing overflows at the reference's row stride."""
    row_length, ind = _connectivity("FixedNumberPreWithReplacement", {"num": num}, num_pre, num_post)
    assert ind.shape[0] == num_pre and row_length.sum() == num * num_post
    valid = np.arange(ind.shape[1])[None, :] < row_length[:, None]
    post = ind[valid]
    pre = np.repeat(np.arange(num_pre), row_length)
    assert post.max() < num_post
    assert np.all(np.bincount(post, minlength=num_post) == num)
    for r in range(0, num_pre, max(1, num_pre // 200)):
        assert np.all(np.diff(ind[r, :row_length[r]].astype(np.int64)) >= 0), f"row {r} is not ascending"
    if num_pre > 1:
        assert stats.chisquare(row_length.astype(np.float64)).pvalue > P_CONNECT
    if num_pre >= 30:           # (with a handful of sources every column holds all of them: nothing to measure)
        # distinct sources per column: E = numPre (1 - (1 - 1/numPre)^num); a generator that reused one word for several
        # draws of a column, or one column's draws for the next, would collapse this
        distinct = np.zeros(num_post, dtype=np.int64)
        pairs = np.unique(post.astype(np.int64) * num_pre + pre)
        np.add.at(distinct, pairs // num_pre, 1)
        expected = num_pre * (1.0 - (1.0 - 1.0 / num_pre) ** num)
        spread = np.sqrt(max(1e-12, num_pre * (1 - 1 / num_pre) ** num * (1 - (1 - 1 / num_pre) ** num)) / num_post)
        assert abs(distinct.mean() - expected) < 5.0 * spread + 1e-9, (distinct.mean(), expected, spread)
        # two columns never share their whole draw
        if num >= 3 and num_pre >= 1000:
            order = np.lexsort((pre, post))
            columns = pre[order].reshape(num_post, num)
            assert len(np.unique(columns, axis=0)) == num_post


def _conv2d_rows(p):
    """Brute force over (pre, post) pairs: a synapse exists where the kernel covers the input pixel, the definition that
    the snippet's row build code (initSparseConnectivitySnippet.h:438-483) enumerates."""
    rows, kernel_index = [], []
    for pre in range(p["conv_ih"] * p["conv_iw"] * p["conv_ic"]):
        in_row, in_col, in_chan = (pre // p["conv_ic"]) // p["conv_iw"], (pre // p["conv_ic"]) % p["conv_iw"], pre % p["conv_ic"]
        row, kern = [], []
        for out_row in range(p["conv_oh"]):
            kr = in_row - (out_row * p["conv_sh"] - p["conv_padh"])
            if not 0 <= kr < p["conv_kh"]:
                continue
            for out_col in range(p["conv_ow"]):
                kc = in_col - (out_col * p["conv_sw"] - p["conv_padw"])
                if not 0 <= kc < p["conv_kw"]:
                    continue
                for out_chan in range(p["conv_oc"]):
                    row.append((out_row * p["conv_ow"] + out_col) * p["conv_oc"] + out_chan)
                    kern.append(((kr * p["conv_kw"] + kc) * p["conv_ic"] + in_chan) * p["conv_oc"] + out_chan)
        rows.append(row)
        kernel_index.append(kern)
    return rows, kernel_index


@pytest.mark.parametrize("shape", [
    dict(conv_kh=3, conv_kw=3, conv_sh=1, conv_sw=1, conv_padh=1, conv_padw=1, conv_ih=8, conv_iw=8, conv_ic=2, conv_oh=8, conv_ow=8, conv_oc=3),
    dict(conv_kh=3, conv_kw=3, conv_sh=1, conv_sw=1, conv_padh=0, conv_padw=0, conv_ih=10, conv_iw=7, conv_ic=1, conv_oh=8, conv_ow=5, conv_oc=4),
    dict(conv_kh=5, conv_kw=3, conv_sh=2, conv_sw=2, conv_padh=2, conv_padw=1, conv_ih=11, conv_iw=9, conv_ic=3, conv_oh=6, conv_ow=5, conv_oc=2),
    dict(conv_kh=2, conv_kw=4, conv_sh=3, conv_sw=2, conv_padh=0, conv_padw=1, conv_ih=9, conv_iw=12, conv_ic=1, conv_oh=3, conv_ow=6, conv_oc=5),
    dict(conv_kh=1, conv_kw=1, conv_sh=1, conv_sw=1, conv_padh=0, conv_padw=0, conv_ih=4, conv_iw=4, conv_ic=3, conv_oh=4, conv_ow=4, conv_oc=3),
])
def test_conv2d_as_sparse_connectivity(shape):
    """Conv2D as SPARSE connectivity with Kernel-initialised weights (initSparseConnectivitySnippet.h:438-497,
    initVarSnippet.h:100-108) against a brute force over every (pre, post) pair: same targets in the same (ascending)
    order, every weight the kernel entry of its (kernel row, kernel column, input channel, output channel); strides above
    one (where some kernel rows have no output row), no padding, and kernels wider than the stride are covered."""
    rng = np.random.default_rng(3)
    kernel = rng.normal(size=(shape["conv_kh"], shape["conv_kw"], shape["conv_ic"], shape["conv_oc"])).astype(np.float32)
    model = _empty_model(1)
    n_pre, n_post = shape["conv_ih"] * shape["conv_iw"] * shape["conv_ic"], shape["conv_oh"] * shape["conv_ow"] * shape["conv_oc"]
    pre = model.add_neuron_population("Pre", n_pre, "LIF", _LIF, {"V": 0.0, "RefracTime": 0.0})
    post = model.add_neuron_population("Post", n_post, "LIF", _LIF, {"V": 0.0, "RefracTime": 0.0})
    s = model.add_synapse_population("S", "SPARSE", pre, post, init_weight_update("StaticPulse", {}, {"g": init_var("Kernel", {"kernel": kernel})}),
                                     init_postsynaptic("DeltaCurr"), init_sparse_connectivity("Conv2D", shape))
    model.build()
    model.load()
    s.pull_connectivity_from_device()
    s.vars["g"].pull_from_device()
    g = s.vars["g"].view.reshape(n_pre, s.row_stride).copy()
    row_length, ind = s.row_length_host.copy(), s.ind_host.copy()
    model.unload()
    rows, kernel_index = _conv2d_rows(shape)
    flat = kernel.reshape(-1)
    assert s.row_stride == -(-shape["conv_kh"] // shape["conv_sh"]) * -(-shape["conv_kw"] // shape["conv_sw"]) * shape["conv_oc"]
    assert max(len(r) for r in rows) <= s.row_stride
    for i, (row, kern) in enumerate(zip(rows, kernel_index)):
        assert row_length[i] == len(row), f"row {i}"
        assert np.array_equal(ind[i, :len(row)], np.asarray(row, dtype=np.uint32)), f"row {i}"
        assert np.array_equal(g[i, :len(row)], flat[kern]), f"row {i}: weights"


@pytest.mark.parametrize("num_post", [1000, 37, 5000])
def test_fixed_probability(num_post):
    """Every (pre, post) pair is an independent Bernoulli(prob) trial: row lengths are Binomial(numPost, prob), every
    column (and so every lane's slice of a row) is hit equally often, rows ascend without repeats."""
    num_pre, prob = 1000, 0.1
    row_length, ind = _connectivity("FixedProbability", {"prob": prob}, num_pre, num_post)
    assert ind.shape[1] == max_row_length("FixedProbability", {"prob": prob}, num_pre, num_post)
    mask = np.arange(ind.shape[1])[None, :] < row_length[:, None]
    for r in range(0, num_pre, 17):
        row = ind[r, :row_length[r]].astype(np.int64)
        assert np.all(np.diff(row) > 0) and (len(row) == 0 or row[-1] < num_post)
    total = int(row_length.sum())
    sd = np.sqrt(num_pre * num_post * prob * (1.0 - prob))
    assert abs(total - num_pre * num_post * prob) < 4.5 * sd
    columns = np.bincount(ind[mask], minlength=num_post)
    assert stats.chisquare(columns).pvalue > P_CONNECT
    lo, hi = int(stats.binom.ppf(1e-3, num_post, prob)), int(stats.binom.ppf(1.0 - 1e-3, num_post, prob))
    obs = np.bincount(np.clip(row_length, lo, hi), minlength=hi + 1)[lo:hi + 1].astype(np.float64)
    cdf = stats.binom.cdf(np.arange(lo, hi + 1), num_post, prob)
    exp = np.diff(np.concatenate(([0.0], cdf[:-1], [1.0]))) * num_pre
    keep = exp >= 5.0
    obs, exp = np.append(obs[keep], obs[~keep].sum()), np.append(exp[keep], exp[~keep].sum())
    assert stats.chisquare(obs[exp > 0], exp[exp > 0]).pvalue > P_CONNECT
    # neighbouring pairs are independent: given that (r, j) exists, (r, j+1) exists with probability prob
    dense = np.zeros((num_pre, num_post), dtype=bool)
    dense[np.repeat(np.arange(num_pre), row_length), ind[mask]] = True
    assert int(dense.sum()) == total
    followed, candidates = int((dense[:, :-1] & dense[:, 1:]).sum()), int(dense[:, :-1].sum())
    assert abs(followed / candidates - prob) < 4.5 * np.sqrt(prob * (1 - prob) / candidates)


def test_fixed_probability_no_autapse_and_extremes():
    n, prob = 2000, 0.05
    row_length, ind = _connectivity("FixedProbabilityNoAutapse", {"prob": prob}, n, n)
    mask = np.arange(ind.shape[1])[None, :] < row_length[:, None]
    rows = np.repeat(np.arange(n), row_length)
    assert not np.any(ind[mask] == rows)
    assert stats.chisquare(np.bincount(ind[mask], minlength=n)).pvalue > P_CONNECT
    row_length, ind = _connectivity("FixedProbability", {"prob": prob}, n, n)
    mask = np.arange(ind.shape[1])[None, :] < row_length[:, None]
    diagonal = int((ind[mask] == np.repeat(np.arange(n), row_length)).sum())
    assert abs(diagonal - n * prob) < 4.5 * np.sqrt(n * prob * (1 - prob))
    # prob = 1: every pair; prob = 0: none
    row_length, ind = _connectivity("FixedProbability", {"prob": 1.0}, 50, 130)
    assert np.all(row_length == 130) and np.array_equal(ind, np.broadcast_to(np.arange(130, dtype=np.uint32), (50, 130)))
    row_length, _ = _connectivity("FixedProbability", {"prob": 0.0}, 50, 130)
    assert np.all(row_length == 0)


def test_row_overflow_is_reported():
    lib = _abi.load()
    _abi.check(lib.gennmi_init(0))
    num_pre, num_post, stride = 64, 1000, 8
    row_length, ind = _device_array(num_pre, np.uint32), _device_array(num_pre * stride, np.uint32)
    overflow = C.c_uint32()
    rc = lib.gennmi_init_sparse_fixed_probability(num_pre, num_post, stride, 0.5, 0, 1, 1, row_length.ptr, ind.ptr, C.byref(overflow))
    assert rc == -2 and overflow.value == num_pre and b"rowStride" in lib.gennmi_last_error()
    assert np.all(row_length.pull_from_device() == stride)
    assert lib.gennmi_init_sparse_fixed_number_post(num_pre, num_post, stride, 9, None, 1, 1, row_length.ptr, ind.ptr, None) == -2
    row_length.free()
    ind.free()


def test_network_initialised_on_the_device_runs():
    """A random network built entirely on the device steps like any other: every spike delivers exactly its row."""
    n, fan_out, steps = 20000, 100, 200
    model = _empty_model(seed=3)
    pop = model.add_neuron_population("N", n, "Izhikevich", {"a": 0.02, "b": 0.2, "c": -65.0, "d": 8.0},
                                      {"V": init_var("Uniform", {"min": -70.0, "max": -50.0}), "U": init_var("Normal", {"mean": -13.0, "sd": 1.0})})
    pop.spike_recording_enabled = True
    model.add_current_source("Drive", "DC", pop, {"amp": 10.0})
    model.add_synapse_population("NN", "SPARSE", pop, pop, init_weight_update("StaticPulse", {}, {"g": init_var("Uniform", {"min": 0.0, "max": 0.2})}),
                                 init_postsynaptic("DeltaCurr"), init_sparse_connectivity("FixedNumberPostWithReplacement", {"num": fan_out}))
    model.build()
    model.load(num_recording_timesteps=steps)
    v0 = pop.vars["V"].pull_from_device()
    assert stats.kstest(v0.astype(np.float64), stats.uniform(-70.0, 20.0).cdf).pvalue > P_VAR
    model.run(steps)
    model.pull_recording_buffers_from_device()
    times, ids = pop.spike_recording_data[0]
    assert len(ids) > n // 2
    delivered = int((times < (steps - 1) * model.dt - 1e-6).sum()) * fan_out
    assert model.synaptic_event_count == delivered
    model.unload()
