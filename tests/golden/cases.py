"""Definitions of the golden cases: small networks of each configuration's shape.  Shared by
make_golden.py (which runs the reference's own CPU backend on them, in the builder container)
and by the tests (which regenerate the same inputs and compare against the stored outputs)."""
from genn_amd import configs


def va_small():
    return configs.vogels_abbott(n=400, steps=300, p=0.1), 50


def potjans_small():
    return configs.potjans(neuron_scale=0.02, connectivity_scale=0.2, steps=400), 50


def izhikevich_small():
    return configs.izhikevich_fanout(n=500, fanout=50, steps=200), 25


def stdp_small():
    return configs.plastic_stdp(n=500, n_src=50, steps=200, fan=60, src_fan=40), 25


def conv_small():
    return configs.conv_toeplitz(h=8, w=8, ic=2, oc=4, steps=100, w_sd=0.6, ioffset=0.4), 25


def va_delay_small():
    # axonal delays: E's ring has 4 slots (longest outgoing delay 3), I's has 6; IE reads the newest slot of a ring
    return configs.vogels_abbott(n=400, steps=300, p=0.1, axonal_delays={"EE": 3, "EI": 1, "IE": 0, "II": 5}), 50


def dense_small():
    return configs.dense_bitmask(), 25


def graded_small():
    return configs.graded(), 25


def reverse_small():
    return configs.reverse(), 25


def stdp_additive_small():
    return configs.plastic_stdp(n=500, n_src=50, steps=200, fan=60, src_fan=40, rule="stdp_additive"), 25


def custom_small():
    # models that are not built in anywhere (an extra neuron state variable, weight-update pre / post variables): they reach
    # the MI355X backend's generated kernels
    return configs.custom_models(), 25


def stdp_delay_small():
    # trace STDP over a projection with an axonal delay (spike times, traces and the weight-update variables then live in
    # the populations' delay slots, neuronUpdateGroupMerged.cc:714-770 copies them from slot to slot) beside a delayed static one:
    # the device library refuses that combination, so on the MI355X backend the model takes generated kernels
    net, snap = stdp_small()
    net.name = "stdp_delay"
    net.syn("EE").axonal_delay_steps = 3
    net.syn("EI").axonal_delay_steps = 1
    return net, snap


def custom_batch1_small():
    # custom_small from other initial values (same matrices): what the second batch of a batched run of custom_small
    # starts from.  The reference's CPU backend has no batches, so every batch of that run is pinned by a run of its own.
    import numpy as np
    from genn_amd import rng
    net, snap = custom_small()
    net.name = "custom_batch1"
    for k, p in enumerate(net.pops):
        p.vars["V"] = (-60.0 + 9.5 * rng.uniform(net.seed, 61 + k, 0, p.n)).astype(np.float32)
        p.vars["A"] = (0.1 * rng.uniform(net.seed, 65 + k, 0, p.n)).astype(np.float32)
    return net, snap


def poisson_input_small():
    # the built-in Poisson neuron (random numbers in simulation code): the fixture holds the reference CPU backend's rasters,
    # of which only the statistics carry over to another generator
    return configs.poisson_input(), 250


def synapse_dynamics_small():
    # weight-update code that runs for every synapse every step (a model of the test driver): generated kernels only
    return configs.synapse_dynamics(), 25


def prev_times_small():
    # weight-update code that reads the PREVIOUS spike times of both ends (prev_st_pre, prev_st_post): populations then keep
    # them, updated before each step from the last step's spike queue
    net = configs.custom_models(timing="prev_timing")
    net.name = "prev_times"
    return net, 25


def dynamic_small():
    # parameters changed while the model runs (setParamDynamic + Runtime::setDynamicParamValue): the drive of the
    # excitatory population twice, the threshold of the inhibitory one, and the time constant of a postsynaptic model, whose
    # code reads only parameters DERIVED from it -- those are computed once, so that change must have no effect.  The
    # MI355X backend bakes parameters into its library descriptors: a model with dynamic ones takes generated kernels
    net, snap = va_small()
    net.name = "dynamic_small"
    net.dynamic = [("neuron", "E", "Ioffset", 100, 0.1), ("ps", "IE", "tau", 150, 20.0), ("neuron", "I", "Vthresh", 180, -52.0),
                   ("neuron", "E", "Ioffset", 220, 0.9)]
    return net, snap


def custom_update_small():
    # custom updates (Runtime::customUpdate): per-neuron, reductions over neurons and batches, per-synapse over SPARSE and
    # DENSE matrices, transpose; kernels generated from the update code on the MI355X backend
    return configs.custom_updates(), 50


def custom_update_static_small():
    # custom updates over a network the device library steps on its resident plan (static weights, no delays, steps queued
    # through Runtime::stepTime): the weights of a static projection decay every 40 steps, one population's potentials are
    # pulled to rest every 25 — the library has to run its queued steps first and rebuild its packed copies of the weights after
    from genn_amd.netspec import Custom
    net, _ = va_small()
    net.name = "custom_update_static"
    net.customs.append(Custom("EEDecay", "Decay", "wu_decay", "EE", params=dict(factor=0.8)))
    net.customs.append(Custom("IRest", "Homeostasis", "decay", "I", params=dict(rest=-60.0, factor=0.25)))
    net.custom_calls += [("Decay", 40), ("Homeostasis", 25)]
    return net, 100


def rewiring_small():
    # custom connectivity updates: synapses removed and added between steps of a learning network
    return configs.rewiring(), 50


def post_events_small():
    # spike-like events of the postsynaptic population (a condition on the target's membrane potential), with reverse output
    return configs.post_events(), 25


def va_double_small():
    # va_small as a double-precision model (ModelSpec::setPrecision): state, weights and accumulators are fp64; the device
    # library's kernels are fp32, so on the MI355X backend the model takes generated kernels
    net, snap = va_small()
    net.name = "va_double"
    net.precision = "double"
    return net, snap


def potjans_poisson_net():
    """10 % of the neurons at 20 % in-degree under the script's own Poisson background, 5 s of model time (rates fixture only)."""
    return configs.potjans(neuron_scale=0.1, connectivity_scale=0.2, steps=50000, poisson=True)


# cases the reference's CPU backend pins directly (fixtures) and that the oracle, a restatement of the built-in models
# with fixed parameters, does not cover
REFERENCE_ONLY = {"va_double_small", "post_events_small", "rewiring_small", "custom_update_small", "custom_update_static_small", "stdp_delay_small", "custom_small", "custom_batch1_small", "dynamic_small", "poisson_input_small", "synapse_dynamics_small", "prev_times_small"}

CASES = {"va_double_small": va_double_small, "post_events_small": post_events_small, "rewiring_small": rewiring_small, "custom_update_small": custom_update_small, "custom_update_static_small": custom_update_static_small, "prev_times_small": prev_times_small, "stdp_delay_small": stdp_delay_small, "synapse_dynamics_small": synapse_dynamics_small, "poisson_input_small": poisson_input_small, "custom_small": custom_small, "custom_batch1_small": custom_batch1_small, "dynamic_small": dynamic_small, "stdp_additive_small": stdp_additive_small, "reverse_small": reverse_small, "graded_small": graded_small, "va_delay_small": va_delay_small, "dense_small": dense_small, "va_small": va_small, "potjans_small": potjans_small, "izhikevich_small": izhikevich_small,
         "stdp_small": stdp_small, "conv_small": conv_small}
