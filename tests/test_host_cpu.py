"""CPU tests of the host side and of the C-ABI library's surface (no device calls)."""
import ctypes as C
import math
import os
import re

import numpy as np
import pytest

from genn_amd import _abi, configs, netgen, rng
from genn_amd.genn_model import GeNNModel, init_postsynaptic, init_weight_update, lit32, field32, model_from_net

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_library_exports_every_declared_symbol():
    header = open(os.path.join(ROOT, "include", "genn_mi355x.h")).read()
    declared = set(re.findall(r"\b(gennmi_[a-z0-9_]+)\s*\(", header))
    assert declared, "no prototypes found in the header"
    lib = _abi.load()
    for name in declared:
        assert hasattr(lib, name), f"{name} is declared in include/genn_mi355x.h but not exported"
    assert declared == set(_abi.SYMBOLS), "ctypes prototype table and header disagree"


def test_struct_layout_matches_the_library():
    sizes = (C.c_size_t * 5)()
    assert _abi.load().gennmi_abi_struct_sizes(C.byref(sizes)) == 0
    assert list(sizes) == [C.sizeof(_abi.Psm), C.sizeof(_abi.Cs), C.sizeof(_abi.NeuronUpdateGroup),
                           C.sizeof(_abi.PresynapticUpdateGroup), C.sizeof(_abi.PostsynapticUpdateGroup)]


def test_error_reporting_without_a_device():
    lib = _abi.load()
    assert lib.gennmi_abi_struct_sizes(None) == -2
    assert b"null" in lib.gennmi_last_error()
    with pytest.raises(_abi.GennmiError):
        _abi.check(lib.gennmi_runner_finalise(None))


def test_literal_and_field_rounding():
    # 0.1 as a literal and as a struct field agree; a value next to a rounding boundary does not
    assert lit32(0.1) == field32(0.1) == np.float32(0.1)
    x = float(np.float32(1.0)) + 2.0 ** -24 + 2.0 ** -40     # just above the midpoint of two floats
    assert field32(x) == np.nextafter(np.float32(1.0), np.float32(2.0))
    assert lit32(x) == np.float32(float("%.9e" % x))
    assert lit32(math.exp(-0.1 / 20.0)) == np.float32("9.950124792e-01")
    assert lit32(0.0) == 0.0 and lit32(-65.0) == np.float32(-65.0)


def test_generators_agree_and_shapes_hold():
    assert np.array_equal(netgen.words(9, 3, 17, 500), rng.words(9, 3, 17, 500))
    assert np.array_equal(netgen.normal_f32(9, 3, 0, 500, 1.0, 2.0), (1.0 + 2.0 * rng.normal(9, 3, 0, 500)).astype(np.float32))
    rl, ind = netgen.fixed_probability(2, 5, 300, 200, 0.1, pad=4)
    assert ind.shape[1] % 4 == 0 and ind.shape[1] >= rl.max()
    assert abs(rl.mean() - 20.0) < 1.5
    for r in range(300):
        row = ind[r, :rl[r]].astype(np.int64)
        assert np.all(np.diff(row) > 0) and (len(row) == 0 or row[-1] < 200)
    rl, ind = netgen.fixed_number_total(2, 6, 50, 40, 1000)
    assert rl.sum() == 1000
    for r in range(50):
        assert np.all(np.diff(ind[r, :rl[r]].astype(np.int64)) >= 0)       # multapses allowed
    rl, ind = netgen.fixed_number_post(2, 7, 10, 1000, 64)
    assert np.all(rl == 64) and ind.shape == (10, 64)
    d = netgen.rows_clipped_normal_delay(2, 8, rl, 64, 15.0, 7.5, 0.0, 42.89)
    assert d.min() >= 0 and d.max() <= 43


def test_full_scale_microcircuit_counts():
    """298,624,465 synapses in 54 non-empty projections, 43 delay slots (userproject/potjans_microcircuit.py:108-133, 181-190)."""
    pops = [l + p for l in configs.PD_LAYERS for p in ("E", "I")]
    total, nonempty = 0, 0
    for trg in pops:
        for src in pops:
            k = int(round(configs.pd_full_num_inputs(src, trg) * float(configs.PD_NUM[trg])))
            total += k
            nonempty += k > 0
    assert total == 298624465 and nonempty == 54
    assert sum(configs.PD_NUM.values()) == 77169
    max_delay = configs.PD_MEAN_DELAY["E"] + configs.PD_DELAY_SD["E"] * configs.PD_NORM_Q9999
    assert int(round(max_delay / 0.1)) == 43


def test_postsynaptic_fusing_and_child_order():
    """Fusing walks incoming projections last-to-first (src/genn/genn/neuronGroup.cc:41-96): the owner of a fused
    outPost is the LAST projection added, and unfused children keep reverse creation order."""
    net = configs.potjans(neuron_scale=0.01, connectivity_scale=0.05, steps=10)
    m = model_from_net(net)
    for n in m.neuron_populations.values():
        assert len(n.fused_psm) == 1
        assert n.fused_psm[0][0] is n.in_syn[-1]
        assert all(s.fused_ps_target is n.in_syn[-1] for s in n.in_syn)
    net = configs.vogels_abbott(n=100, steps=10, p=0.1)
    m = model_from_net(net)
    e = m.neuron_populations["E"]
    assert [grp[0].name for grp in e.fused_psm] == ["IE", "EE"]


def test_unsupported_models_fail_loudly():
    m = GeNNModel("float", "x")
    with pytest.raises(NotImplementedError):
        m.add_neuron_population("p", 10, "TraubMiles", {}, {})
    with pytest.raises(NotImplementedError):
        init_weight_update("PiecewiseSTDP")
    with pytest.raises(NotImplementedError):
        init_postsynaptic("ExpCond")
    with pytest.raises(NotImplementedError):
        GeNNModel("double", "x")
    p = m.add_neuron_population("p", 10, "LIF", {}, {})
    with pytest.raises(RuntimeError):
        m.load()           # build() first, as in the reference


def test_bench_refuses_more_than_one_gpu():
    import subprocess
    import sys
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert r.returncode != 0 and "one GPU" in (r.stderr + r.stdout)


def test_philox_known_answers():
    """The generator under the on-device initialisation snippets, through the library's host entry point and the numpy
    restatement the GPU tests compare device output with: both must give the published known-answer vectors."""
    import ctypes as C
    from philox_ref import KNOWN_ANSWERS, philox4x32
    lib = _abi.load()
    for counter, key, want in KNOWN_ANSWERS:
        out = (C.c_uint32 * 4)()
        assert lib.gennmi_philox4x32(C.byref((C.c_uint32 * 4)(*counter)), C.byref((C.c_uint32 * 2)(*key)), C.byref(out)) == 0
        assert tuple(out) == want
        assert tuple(int(w) for w in philox4x32(*counter, *key)) == want


def test_max_row_length_follows_the_snippets():
    """Row strides of the built-in connectivity snippets against the known answers of the reference's unit test for
    binomialInverseCDF (tests/unit/binomial.cc:15-35: square matrices of 1, 1000 and 10^6 neurons at three probabilities)."""
    from genn_amd.genn_model import max_row_length
    table = {0.02: (1, 47, 20897), 0.1: (1, 153, 101914), 1.0: (1, 1000, 1000000)}
    for prob, want in table.items():
        for size, stride in zip((1, 1000, 1000000), want):
            assert max_row_length("FixedProbability", {"prob": prob}, size, size) == stride
    assert max_row_length("FixedNumberPostWithReplacement", {"num": 37}, 100, 100) == 37
    assert max_row_length("OneToOne", {}, 100, 100) == 1
