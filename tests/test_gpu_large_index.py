"""A projection whose padded synapse count exceeds 2^32 - 1 (the reference switches its synapse-index type to 64 bits there,
backendBase.cc:503-522): 1,100,000 rows of 4,096 targets = 4.5 x 10^9 synapses, 36 GB of `ind` and `g`, built by the
device-side initialisation (no host copy exists) and stepped through both presynaptic paths — a handful of spikes (scatter
kernel) and a burst (tile kernel) — with spiking rows on either side of the 2^32 boundary (row 1,048,576 starts at synapse
2^32 exactly).  Checked against sums recomputed on the host from the spiking rows alone, pulled as slices.

The CPU oracle cannot hold this matrix in the time a test has; what is pinned is the indexing, which is all that changes
with size.
"""
import numpy as np
import pytest

from genn_amd.genn_model import (GeNNModel, init_postsynaptic, init_sparse_connectivity, init_var, init_weight_update)

pytestmark = pytest.mark.gpu

LIF_SILENT = {"C": 1.0, "TauM": 20.0, "Vrest": -60.0, "Vreset": -60.0, "Vthresh": 1e9, "Ioffset": 0.0, "TauRefrac": 5.0}
N_SRC, N_TRG, NUM = 1_100_000, 1_000_000, 4096
BOUNDARY = (1 << 32) // NUM            # first row whose synapses lie beyond 2^32


def test_rows_beyond_32_bit_synapse_ids_are_delivered():
    few = np.array([0, 5, BOUNDARY - 1, BOUNDARY, BOUNDARY + 1, N_SRC - 1])
    rng = np.random.default_rng(12)
    burst = np.unique(np.concatenate([rng.integers(0, N_SRC, 1500), [1, BOUNDARY - 2, BOUNDARY + 2, N_SRC - 2]]))
    burst = burst[~np.isin(burst, few)]
    fire = np.full(N_SRC, -1)
    fire[few] = 0
    fire[burst] = 1

    model = GeNNModel("float", "large_index", batch_size=1, dt=1.0)
    model.seed = 77
    fires = fire >= 0
    end = np.cumsum(fires).astype(np.uint32)
    start = (end - fires).astype(np.uint32)
    src = model.add_neuron_population("S", N_SRC, "SpikeSourceArray", {}, {"startSpike": start[None, :], "endSpike": end[None, :]})
    src.set_extra_global_param("spikeTimes", np.concatenate([fire[fires].astype(np.float32), [0.0]]).astype(np.float32))
    trg = model.add_neuron_population("T", N_TRG, "LIF", LIF_SILENT, {"V": -60.0, "RefracTime": 0.0})
    s = model.add_synapse_population("ST", "SPARSE", src, trg,
                                     init_weight_update("StaticPulse", {}, {"g": init_var("Uniform", {"min": 0.25, "max": 1.0})}),
                                     init_postsynaptic("DeltaCurr"), init_sparse_connectivity("FixedNumberPostWithReplacement", {"num": NUM}))
    model.build()
    model.load()
    assert s.row_stride == NUM and N_SRC * s.row_stride > 0xFFFFFFFF
    info = model.runner_info()
    assert not info["resident_plan"]

    def rows(ids):
        out = np.zeros(N_TRG)
        events = 0
        for i in ids:
            n = int(s.vars["rowLength"].pull_slice(i, 1)[0])
            assert n == NUM
            ind = s.vars["ind"].pull_slice(int(i) * NUM, n)
            g = s.vars["g"].pull_slice(int(i) * NUM, n).astype(np.float64)
            assert ind.max() < N_TRG and np.all(np.diff(ind.astype(np.int64)) >= 0)
            assert g.min() >= 0.25 and g.max() <= 1.0
            np.add.at(out, ind, g)
            events += n
        return out, events

    total_events = 0
    for step, ids in ((1, few), (2, burst)):
        # the step after a source's spike time delivers its row: neurons (spikes of `step - 1`), then synapses
        while model.timestep < step:
            model.update_synapses()
            model.update_neurons()
        model.update_synapses()
        got = s.vars["outPost"].pull_from_device().astype(np.float64)
        want, events = rows(ids)
        total_events += events
        peak = float(want.max())
        assert peak > 0.0
        assert np.abs(got - want).max() <= 1e-5 * max(1.0, peak), f"step {step}: {len(ids)} spiking rows"
        assert model.synaptic_event_count == total_events
        model.update_neurons()
    model.unload()
