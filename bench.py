#!/usr/bin/env python3
"""Benchmark of the per-timestep hot path on one MI355X.

Workload (default): the full-scale cortical microcircuit — 77,169 LIF neurons in 8 populations,
298,624,465 synapses in 54 SPARSE projections with fp32 weights and uint8 dendritic delays into a
43-slot ring, DC background, dt = 0.1 ms.  A "step" is one simulation timestep
(updateSynapses + updateNeurons).  Inputs are synthetic (repo-owned seeded generator) and already
resident in HBM when the timed region starts.

Prints ONE JSON line: whole-job synaptic events per second, plus
  roofline      the dominant kernel against the HBM roofline (algorithmic bytes per event
                x events per launch / average launch duration from HIP events on the kernel's stream)
  cpu_baseline  the single-threaded CPU oracle timed on this host on a bounded sample of the same network
  steady_state  (short runs only) the same network stepped on in the same process — 2,000 untimed steps, then 10,000
                timed ones — with its own roofline: a run of a few steps from t = 0 times the launch's start-up and the
                synchronous burst every cold start of the network goes through, not the running network
  secondary     (default workload only) the bandwidth-bound case beside the latency-bound headline: configuration 3 —
                10^6 Izhikevich neurons, 10^9 synapses, its own noise array — for 1,000 steps (1 s simulated), with the
                presynaptic kernels' fraction of the HBM roofline
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
# algorithmic bytes per synaptic event: ind 4 + g 4 + fp32 read-modify-write of the target 8 (+ 1 delay byte)
BYTES_PER_EVENT = {"dense": 4,          # one weight read per (spike, target); outPost is read and written once per target and step
                   "static": 16, "static_delay": 17, "stdp_trace": 28, "conv2d": 8}
# HBM bytes per launch of the dominant kernel, from hardware counters (rocprofv3 --pmc FETCH_SIZE, then WRITE_SIZE, each
# scaled by what the same counter reads for the library's 256 MiB copy kernel); recorded with the commands that
# produced them in profiles/<kernel>_<workload>.md.  A counter run is a separate invocation of this script, so the figure
# is only attached to a run of the very command line it was measured on (same workload, steps and warm-up: the network,
# its seed and therefore its activity are then identical); any other run reports null.
# The kernel's source is named with a digest: a figure measured on another version of the kernel is not attached.
MEASURED_TRAFFIC_BYTES = {
    ("potjans", 20, 5): {"plan": "resident", "bytes_per_launch": 155216672,
                         "kernel_source": ("genn_amd/csrc/genn_mi355x_resident_kernels.h", "861e3def22045d8a"),
                         "source": "rocprofv3 --pmc FETCH_SIZE (67692.56 x 2 KiB) + WRITE_SIZE (16193.66 x 1 KiB) of the timed 20-step "
                                   "launch, profiles/residentKernel_potjans_full.md"},
    ("conv", 1000, 100): {"plan": "stepped", "requires": "conv_step_in_one_launch", "bytes_per_launch": 66118287,
                          "kernel_source": ("genn_amd/csrc/genn_mi355x_conv_step_kernels.h", "b33aec4cfae473d9"),
                          "source": "rocprofv3 --pmc FETCH_SIZE (18888.04 x 2 KiB) + WRITE_SIZE (26792.56 x 1 KiB), average over the "
                                    "run's 1,100 launches, profiles/convStepKernel_conv_batch16.md"},
}
FP32_MFMA_PEAK_TFLOPS = 157.3


def source_digest(path):
    import hashlib
    with open(os.path.join(ROOT, path), "rb") as f:
        return hashlib.sha256(f.read()).hexdigest()[:16]


def build_net(name, steps):
    from genn_amd import configs
    if name == "potjans":
        return configs.potjans(steps=steps), "C2 potjans_microcircuit 77169 neurons 298.6M synapses dt=0.1ms"
    if name == "potjans_poisson":
        return configs.potjans(steps=steps, poisson=True), "C2 potjans_microcircuit 77169 neurons 298.6M synapses dt=0.1ms, PoissonExp background (Philox)"
    if name == "potjans_small":
        return configs.potjans(neuron_scale=0.1, connectivity_scale=1.0, steps=steps), "potjans 10% neurons full in-degree"
    if name == "va":
        return configs.vogels_abbott(steps=steps), "C1 balanced LIF 4000 neurons p=0.02 dt=0.1ms"
    if name == "dense":
        return configs.dense_layer(steps=steps), "dense layer 8192 Poisson sources (50 Hz) -> 8192 LIF, DENSE individual weights, dt=1ms"
    if name == "izh":
        # the configuration's own noise array: one row of 10^6 values per step for 1 s simulated (4 GB); a run of more
        # than 1000 steps starts over at its first row
        return (configs.izhikevich_fanout(steps=steps, noise_steps=min(steps, 1000)),
                "C3 izhikevich 1e6 neurons fanout 1000 dt=1ms, per-step noise array of min(steps, 1000) rows")
    if name == "izh_small":
        return configs.izhikevich_fanout(n=100_000, fanout=1000, steps=steps, noise_steps=64), "izhikevich 1e5 neurons fanout 1000"
    if name == "stdp":
        return configs.plastic_stdp(steps=steps), "C4 plastic STDP 100k neurons fanout 500 dt=1ms"
    if name == "conv":
        import copy
        import numpy as np
        B = 16
        nets = [configs.conv_toeplitz(steps=steps, batch_index=b, w_sd=0.1, ioffset=0.3) for b in range(B)]
        times = np.concatenate([n.pop("In").spike_times for n in nets])
        offs = np.cumsum([0] + [len(n.pop("In").spike_times) for n in nets])
        net = copy.deepcopy(nets[0])
        net.pop("In").vars = {"startSpike": np.stack([n.pop("In").vars["startSpike"] + offs[b] for b, n in enumerate(nets)]).astype(np.uint32),
                              "endSpike": np.stack([n.pop("In").vars["endSpike"] + offs[b] for b, n in enumerate(nets)]).astype(np.uint32)}
        net.pop("In").spike_times = times
        net.batch_size = B
        net.batch_nets = nets
        return net, "C5 conv2d 3x3 64x64x16 -> 64x64x32 TOEPLITZ, batch 16, dt=1ms"
    raise SystemExit(f"unknown workload {name}")


def bench_init(args):
    """--workload init_izhikevich: on-device initialisation at the size of the 10^6-neuron configuration — 10^6 rows of
    1000 ascending targets (FixedNumberPostWithReplacement) and 10^9 uniform weights.  A step builds both arrays once
    (8 GB written); connectivity and weights are timed separately with the host clock around synchronous calls."""
    import ctypes as C
    import numpy as np
    from genn_amd import _abi
    from genn_amd.genn_model import Array
    lib = _abi.load()
    _abi.check(lib.gennmi_init(0))
    num, fan_out = 1_000_000, 1000
    row_length, ind, g = Array(num, np.uint32, device_only=True), Array(num * fan_out, np.uint32, device_only=True), Array(num * fan_out, np.float32, device_only=True)
    params = (C.c_double * 4)(0.0, 0.5, 0.0, 0.0)
    steps = min(args.steps, 20)
    warmup = min(args.warmup, 2)
    t_conn = t_var = 0.0
    for it in range(warmup + steps):
        t0 = time.perf_counter()
        _abi.check(lib.gennmi_init_sparse_fixed_number_post(num, num, fan_out, fan_out, None, 1234, 1 + it, row_length.ptr, ind.ptr, None))
        _abi.check(lib.gennmi_synchronize())
        t1 = time.perf_counter()
        _abi.check(lib.gennmi_init_var(g.ptr, _abi.ELEMENT_TYPES["float32"], num * fan_out, _abi.INIT_SNIPPETS["Uniform"], C.byref(params), 1234, 1000 + it))
        _abi.check(lib.gennmi_synchronize())
        t2 = time.perf_counter()
        if it >= warmup:
            t_conn += t1 - t0
            t_var += t2 - t1
    # spot check of the last build: a block of rows is ascending and in range
    sample = np.empty(4096 * fan_out, dtype=np.uint32)
    _abi.check(lib.gennmi_memcpy_from_device(sample.ctypes.data_as(C.c_void_p), ind.ptr, sample.nbytes))
    rows = sample.reshape(4096, fan_out).astype(np.int64)
    assert np.all(np.diff(rows, axis=1) >= 0) and rows.max() < num
    synapses = num * fan_out
    per_step = (t_conn + t_var) / steps
    out = {"metric": "synapses_initialised_per_s", "value": round(synapses / per_step, 1), "unit": "synapses/s", "n_gpus": 1,
           "steps": steps, "warmup": warmup, "ms_per_step": round(per_step * 1e3, 3), "higher_is_better": True, "scaling": "weak",
           "vs_baseline": None, "dtype": "u32+f32", "data": "synthetic",
           "config": {"workload": "on-device initialisation, 10^6 x 1000 FixedNumberPostWithReplacement + Uniform weights", "synapses": synapses},
           "connectivity_ms": round(t_conn / steps * 1e3, 3), "weights_ms": round(t_var / steps * 1e3, 3),
           "roofline": {"bound": "hbm", "kernel": "fixedNumberPostKernel (4 B written per synapse)", "achieved": round(4.0 * synapses / (t_conn / steps) / 1e9, 1),
                        "peak": 8000.0, "unit": "GB/s", "frac": round(4.0 * synapses / (t_conn / steps) / 8e12, 4), "traffic": None,
                        "weights_kernel": {"kernel": "initVarKernel<float>", "achieved": round(4.0 * synapses / (t_var / steps) / 1e9, 1),
                                           "frac": round(4.0 * synapses / (t_var / steps) / 8e12, 4)}},
           "cpu_baseline": None}
    print(json.dumps(out))


def bench_procedural(args, stored, steps=None, warmup=None, profile_steps=None):
    """--workload izh_procedural / izh_stored (the latter is also the default run's `secondary` block): the 10^6-neuron, 10^9-synapse Izhikevich network with its connectivity and
    weights regenerated for every spike (PROCEDURAL: nothing stored), or its stored twin built on the device from the same
    seed (SPARSE).  800,000 excitatory and 200,000 inhibitory neurons; every neuron has 800 + 200 targets
    (FixedNumberPostWithReplacement per target population), weights U[0, 0.5) from excitatory and U[-1, 0) from inhibitory
    rows; DeltaCurr input; a cycled array of U[0, 5) noise."""
    import numpy as np
    from genn_amd import netgen
    from genn_amd.genn_model import GeNNModel, init_postsynaptic, init_sparse_connectivity, init_var, init_weight_update
    n_e, n_i, rows = 800_000, 200_000, 8
    t0 = time.time()
    model = GeNNModel("float", "izh_procedural", dt=1.0)
    model.seed = 777
    izh = dict(a=0.02, b=0.2, c=-65.0, d=8.0)
    pops = {"E": model.add_neuron_population("E", n_e, "Izhikevich", izh, {"V": -65.0, "U": -13.0}),
            "I": model.add_neuron_population("I", n_i, "Izhikevich", izh, {"V": -65.0, "U": -13.0})}
    for k, (name, n) in enumerate((("E", n_e), ("I", n_i))):
        cs = model.add_current_source(name + "_noise", "ArrayNoise", pops[name])
        cs.set_extra_global_param("noise", netgen.uniform_f32(777, 12 + k, 0, rows * n, 5.0, 0.0).reshape(rows, n))
        pops[name].spike_recording_enabled = True
    matrix = "SPARSE" if stored else "PROCEDURAL"
    for src, lo, hi in (("E", 0.0, 0.5), ("I", -1.0, 0.0)):
        for trg, num in (("E", 800), ("I", 200)):
            model.add_synapse_population(src + trg, matrix, pops[src], pops[trg],
                                         init_weight_update("StaticPulse", {}, {"g": init_var("Uniform", {"min": lo, "max": hi})}),
                                         init_postsynaptic("DeltaCurr"), init_sparse_connectivity("FixedNumberPostWithReplacement", {"num": num}))
    steps = args.steps if steps is None else steps
    warmup = args.warmup if warmup is None else warmup
    profile_steps = args.profile_steps if profile_steps is None else profile_steps
    model.build()
    model.load(num_recording_timesteps=warmup + steps)
    model.synchronize()
    load_s = time.time() - t0
    model.run(warmup)
    model.synchronize()
    ev0 = model.synaptic_event_count
    t0 = time.perf_counter()
    model.run(steps)
    model.synchronize()
    wall = time.perf_counter() - t0
    events = model.synaptic_event_count - ev0
    model.pull_recording_buffers_from_device()
    rates = {name: round(len(p.spike_recording_data[0][1]) / p.num_neurons / ((warmup + steps) / 1000.0), 3) for name, p in pops.items()}
    roofline = None
    if profile_steps > 0:
        model.set_timing(True)
        evp0 = model.synaptic_event_count
        model.run(profile_steps)
        model.synchronize()
        st = model.kernel_stats()
        evp = model.synaptic_event_count - evp0
        avg_s = st["presyn_seconds"] / max(1, st["presyn_launches"])
        # algorithmic bytes per event: the fp32 read-modify-write of outPost, plus the stored index and weight if there are any
        bpe = 16 if stored else 8
        achieved = evp / max(1, st["presyn_launches"]) * bpe / avg_s / 1e9
        roofline = {"bound": "hbm", "kernel": "presynapticUpdateKernel + presynapticTileKernel (every step launches both; one of them takes the step)" if stored else "presynapticProceduralKernel",
                    "achieved": round(achieved, 3), "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBS, 6), "traffic": None,
                    "bytes_per_event": bpe, "events_per_launch": round(evp / max(1, st["presyn_launches"]), 1), "avg_launch_us": round(avg_s * 1e6, 3),
                    "events_per_s_in_kernel": round(evp / st["presyn_seconds"], 1) if st["presyn_seconds"] else None,
                    "neuron_kernel_avg_us": round(st["neuron_seconds"] / max(1, st["neuron_launches"]) * 1e6, 3)}
    model.unload()
    return {
        "metric": "synaptic_events_per_s", "value": round(events / wall, 1), "unit": "events/s", "n_gpus": 1, "steps": steps,
        "warmup": warmup, "ms_per_step": round(wall / steps * 1e3, 6), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": "10^6 Izhikevich neurons, 10^9 synapses, " + ("stored on the device (SPARSE, built there)" if stored else "PROCEDURAL (regenerated per spike)"),
                   "neurons": n_e + n_i, "synapses": (n_e + n_i) * 1000, "dt_ms": 1.0, "seed": 777},
        "gsop_per_s": round(events / wall / 1e9, 4), "wall_s_per_sim_s": round(wall / (steps / 1000.0), 4),
        "events_per_step": round(events / steps, 1), "firing_rates_hz": rates, "setup_s": {"build_and_load": round(load_s, 2)},
        "roofline": roofline, "cpu_baseline": None}


def run_net_workload(args, workload, steps, warmup, profile_steps, with_cpu, with_steady):
    """One host-generated network: load, warm-up, timed region, per-kernel pass, (running-network block), (CPU baseline).
    Returns the record of the run."""
    import numpy as np
    from genn_amd.genn_model import model_from_net

    total_steps = warmup + steps + profile_steps
    t0 = time.time()
    net, label = build_net(workload, total_steps)
    gen_s = time.time() - t0
    num_neurons = sum(p.n for p in net.pops)
    num_synapses = sum(s.num_synapses for s in net.syns)
    kinds = {(s.matrix if s.matrix in ("conv2d", "dense", "bitmask") else s.wum) for s in net.syns}
    bytes_per_event = max(BYTES_PER_EVENT[k] for k in kinds) if len(kinds) == 1 else None

    t0 = time.time()
    batch = getattr(net, "batch_size", 1)
    model = model_from_net(net, batch_size=batch, record=True)
    model.load(num_recording_timesteps=warmup + steps)
    model.synchronize()
    load_s = time.time() - t0

    # ---- warm-up (also captures the step graph; the events are recorded around it too, so that creating them and
    # recording for the first time — 30 us of host time — is not part of the timed region), then the timed region
    model.stream_mark(0)
    model.run(warmup)
    model.stream_mark(1)
    model.synchronize()
    ev0 = model.synaptic_event_count
    t0 = time.perf_counter()
    model.stream_mark(0)
    model.run(steps)
    model.stream_mark(1)
    model.synchronize()
    wall = time.perf_counter() - t0
    region_s = model.stream_elapsed()          # HIP events on the runner's stream around the timed region
    events = model.synaptic_event_count - ev0
    events_with_warmup = events + ev0

    model.pull_recording_buffers_from_device()
    rates = {}
    for p in net.pops:
        data = model.neuron_populations[p.name].spike_recording_data
        rates[p.name] = round(sum(len(ids) for _, ids in data) / batch / p.n / ((warmup + steps) * net.dt / 1000.0), 3)

    # ---- per-kernel durations: the same graph replay with HIP event nodes between the kernels of every step
    # (events on the runner's stream; durations are those of back-to-back execution)
    roofline = None
    info = model.runner_info()
    if profile_steps > 0:
        model.set_timing(True)
        evp0 = model.synaptic_event_count
        model.run(profile_steps)
        model.synchronize()
        st = model.kernel_stats()
        evp = model.synaptic_event_count - evp0
        model.set_timing(False)
        bpe = bytes_per_event or max(BYTES_PER_EVENT[k] for k in kinds)
        neuron_bytes = batch * sum(p.n * (0 if p.model == "ssa" else 32) for p in net.pops)     # 32 B per LIF/Izhikevich update (state + one PSM), every batch
        if info["resident_plan"]:
            # the timed region is ONE launch of residentKernel that performs all K steps and nothing else, so HIP events
            # around the region give that launch's duration; a launch moves K steps' worth of
            # algorithmic bytes
            achieved = (events * bpe + neuron_bytes * steps) / region_s / 1e9
            roofline = {"bound": "hbm", "kernel": "residentKernel (all timesteps of the timed region in one launch)",
                        "achieved": round(achieved, 3), "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBS, 6),
                        "traffic": None, "bytes_per_event": bpe, "events_per_launch": events, "steps_per_launch": steps,
                        "neuron_bytes_per_launch": neuron_bytes * steps, "avg_launch_us": round(region_s * 1e6, 3),
                        "us_per_step": round(region_s / steps * 1e6, 3),
                        "avg_launch_us_one_step_per_launch": round(st["step_seconds"] / max(1, st["step_launches"]) * 1e6, 3) if st["step_launches"] else None}
        elif info["single_launch_step"]:
            # the timed region consists of this kernel only (one launch per step, back to back inside the replayed
            # graphs, plus one 1-thread node per 100 steps), so HIP events around the region give its average duration
            avg_s = region_s / steps
            ev_per_launch = events / steps
            achieved = (ev_per_launch * bpe + neuron_bytes) / avg_s / 1e9
            roofline = {"bound": "hbm", "kernel": "stepFusedKernel (presynaptic + neuron update of one timestep)",
                        "achieved": round(achieved, 3), "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBS, 6),
                        "traffic": None, "bytes_per_event": bpe, "events_per_launch": round(ev_per_launch, 1),
                        "neuron_bytes_per_launch": neuron_bytes, "avg_launch_us": round(avg_s * 1e6, 3),
                        "avg_launch_us_individually_launched": round(st["step_seconds"] / max(1, st["step_launches"]) * 1e6, 3)}
        elif info["conv_step_in_one_launch"]:
            # the timed region consists of this kernel only (the layer on the matrix cores, the postsynaptic and neuron model on its
            # accumulators, the source population's update in blocks of the same launch), so HIP events around the region give
            # its average duration; bytes by the event accounting (8 B per event: the target's read-modify-write) plus the state
            avg_s = region_s / steps
            ev_per_launch = events / steps
            achieved = (ev_per_launch * bpe + neuron_bytes) / avg_s / 1e9
            c = [s_ for s_ in net.syns if s_.matrix == "conv2d"][0].conv
            flops = 2.0 * batch * c["conv_oh"] * c["conv_ow"] * c["conv_kh"] * c["conv_kw"] * c["conv_ic"] * c["conv_oc"]
            roofline = {"bound": "hbm", "kernel": "convStepKernel (Conv2D on the matrix cores + neuron update of one timestep)",
                        "achieved": round(achieved, 3), "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBS, 6),
                        "traffic": None, "bytes_per_event": bpe, "events_per_launch": round(ev_per_launch, 1),
                        "neuron_bytes_per_launch": neuron_bytes, "avg_launch_us": round(avg_s * 1e6, 3),
                        "avg_launch_us_individually_launched": round(st["step_seconds"] / max(1, st["step_launches"]) * 1e6, 3),
                        "mfma": {"bound": "mfma", "achieved": round(flops / avg_s / 1e12, 3), "peak": FP32_MFMA_PEAK_TFLOPS, "unit": "TFLOP/s",
                                 "frac": round(flops / avg_s / 1e12 / FP32_MFMA_PEAK_TFLOPS, 4), "flops_per_launch": flops}}
        elif st["presyn_launches"]:
            avg_s = st["presyn_seconds"] / st["presyn_launches"]
            ev_per_launch = evp / st["presyn_launches"]
            achieved = ev_per_launch * bpe / avg_s / 1e9
            navg = st["neuron_seconds"] / max(1, st["neuron_launches"])
            # (the timed pass launches every kernel on its own so that each has an event pair; the untimed region combines the
            # synaptic kernels of a step into one launch where the runner's plan says so)
            if kinds == {"dense"}:
                kernel = "presynapticDenseKernel"
            elif info["conv_on_matrix_cores"]:
                kernel = "presynapticConvMfmaKernel (busy steps) + presynapticUpdateKernel (quiet steps)"
            elif info["combined_synapse_launch"]:
                kernel = ("presynapticUpdateKernel + presynapticTileKernel, launched separately in this timed pass; the untimed region runs them"
                          + (" and the postsynaptic pass" if info["postsynaptic_in_combined_launch"] else "") + " as one synapseCombinedKernel launch per step")
            else:
                kernel = "presynapticUpdateKernel"
            roofline = {"bound": "hbm", "kernel": kernel, "achieved": round(achieved, 3),
                        "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBS, 6), "traffic": None,
                        "bytes_per_event": bpe, "events_per_launch": round(ev_per_launch, 1), "avg_launch_us": round(avg_s * 1e6, 3),
                        "neuron_kernel_avg_us": round(navg * 1e6, 3), "neuron_kernel_gbs": round(neuron_bytes / navg / 1e9, 3)}
            if st["postsyn_launches"]:
                roofline["postsyn_kernel_avg_us"] = round(st["postsyn_seconds"] / st["postsyn_launches"] * 1e6, 3)
            if info["conv_on_matrix_cores"]:
                # the layer as a GEMM per batch and step: (output pixels) x (kh kw ic) x (output channels), fp32 MFMA; every
                # step of this workload is a busy one, so the presynaptic time is the matrix-core kernel's
                c = [s_ for s_ in net.syns if s_.matrix == "conv2d"][0].conv
                flops = 2.0 * batch * c["conv_oh"] * c["conv_ow"] * c["conv_kh"] * c["conv_kw"] * c["conv_ic"] * c["conv_oc"]
                roofline["mfma"] = {"bound": "mfma", "kernel": "presynapticConvMfmaKernel", "achieved": round(flops / avg_s / 1e12, 3), "peak": FP32_MFMA_PEAK_TFLOPS,
                                    "unit": "TFLOP/s", "frac": round(flops / avg_s / 1e12 / FP32_MFMA_PEAK_TFLOPS, 4), "flops_per_launch": flops}
    if args.yardstick_mib > 0:
        from genn_amd.genn_model import Array
        count = args.yardstick_mib * (1 << 20) // 4
        a, b = Array(count, np.float32, fill=1.0), Array(count, np.float32)
        for _ in range(5):
            b.copy_on_device(a)
        a.free(); b.free()
    measured = MEASURED_TRAFFIC_BYTES.get((workload, steps, warmup))
    if roofline is not None and measured is not None and measured["plan"] == ("resident" if info["resident_plan"] else "stepped") \
            and info.get(measured.get("requires", "finalised"), True):
        if source_digest(measured["kernel_source"][0]) == measured["kernel_source"][1]:
            roofline["traffic"] = measured["bytes_per_launch"]
            roofline["traffic_source"] = measured["source"]
        else:
            roofline["traffic_source"] = "not attached: " + measured["kernel_source"][0] + " has changed since the counters were read"

    # ---- the running network: short runs only (see the module docstring)
    steady = None
    if with_steady and args.steady_steps > 0 and steps < 1000:
        model.run(args.steady_warmup)
        model.synchronize()
        ev0s = model.synaptic_event_count
        t0 = time.perf_counter()
        model.stream_mark(0)
        model.run(args.steady_steps)
        model.stream_mark(1)
        model.synchronize()
        wall_s = time.perf_counter() - t0
        region = model.stream_elapsed()
        ev_s = model.synaptic_event_count - ev0s
        bpe = bytes_per_event or max(BYTES_PER_EVENT[k] for k in kinds)
        nbytes = batch * sum(p.n * (0 if p.model == "ssa" else 32) for p in net.pops)
        achieved = (ev_s * bpe + nbytes * args.steady_steps) / region / 1e9
        steady = {"steps": args.steady_steps, "warmup": args.steady_warmup, "us_per_step": round(wall_s / args.steady_steps * 1e6, 3),
                  "events_per_s": round(ev_s / wall_s, 1), "gsop_per_s": round(ev_s / wall_s / 1e9, 4),
                  "events_per_step": round(ev_s / args.steady_steps, 1),
                  "wall_s_per_sim_s": round(wall_s / (args.steady_steps * net.dt / 1000.0), 4),
                  "roofline": {"bound": "hbm", "kernel": ("residentKernel (one launch for all steps of the block)" if info["resident_plan"] else
                                                          "all kernels of the block's steps (hipGraph replay)"),
                               "achieved": round(achieved, 3), "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBS, 6),
                               "avg_launch_us": round(region * 1e6, 3), "us_per_step": round(region / args.steady_steps * 1e6, 3),
                               "bytes_per_event": bpe, "events_per_launch": ev_s, "neuron_bytes_per_launch": nbytes * args.steady_steps, "traffic": None}}
    model.unload()

    # ---- CPU baseline: the single-threaded oracle on the same network, bounded sample from t = 0
    cpu = None
    if with_cpu:
        from oracle.genn_cpu import OracleNet
        # the reference's CPU backend (and the oracle) has no batch dimension: batch 0 is timed and the figure is per batch
        oracle = OracleNet(net.batch_nets[0] if batch > 1 else net)
        # activity is not stationary (silent start, bursts), so the sample is bounded by time, not sized from a probe:
        # blocks of steps until ~12 s of CPU work
        # (the sample does not depend on --steps: a run of a few steps still gets a baseline worth the name)
        cpu_budget_s, block = 12.0, 10
        limit = args.cpu_steps or (1 << 62)
        cpu_steps, cpu_wall = 0, 0.0
        while cpu_steps < limit and (args.cpu_steps or cpu_wall < cpu_budget_s):
            n = min(block, limit - cpu_steps)
            t0 = time.perf_counter()
            oracle.run(n)
            cpu_wall += time.perf_counter() - t0
            cpu_steps += n
            if cpu_wall < 1.0:
                block = min(block * 2, 2000)
        cpu_events = oracle.events()
        probe = 0
        cpu = {"value": round(cpu_events / cpu_wall, 1), "unit": "events/s", "cores": 1, "kind": "port",
               "sample": f"steps {probe}..{probe + cpu_steps} of the same network from t=0 ({cpu_events} events in {cpu_wall:.2f} s)",
               "wall_s_per_sim_s": round(cpu_wall / (cpu_steps * net.dt / 1000.0), 3),
               "host_cores": os.cpu_count()}
        oracle.close()

    # ---- the same network on the reference's OWN SingleThreadedCPU backend (generated code compiled -O3), where
    # the prebuilt driver exists: wall-clock of its Runtime::stepTime loop over a bounded number of steps
    if cpu is not None and args.reference_steps > 0 and batch == 1:
        driver = os.path.join(ROOT, "oracle", "_ref", "ref_driver")
        if os.path.exists(driver):
            import re
            import shutil
            import subprocess
            import tempfile
            from genn_amd.netspec import write_netspec
            tmp = tempfile.mkdtemp(prefix="bench_ref_")
            try:
                spec, work, out_dir = (os.path.join(tmp, d) for d in ("spec", "work", "out"))
                os.makedirs(work); os.makedirs(out_dir)
                # (a per-step noise array holds as many rows as it holds: the driver reads one per step)
                rows = [c.noise.size // net.pop(c.pop).n for c in net.css if getattr(c, "noise", None) is not None]
                old_steps, net.steps, net.snap = net.steps, min([args.reference_steps] + rows), 0
                write_netspec(net, spec)
                net.steps = old_steps
                res = subprocess.run([driver, spec, work, out_dir, "--cxxflags=-O3"], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=600)
                m = re.search(r"stepping loop ([0-9.eE+-]+) s for (\d+) steps", res.stdout)
                if res.returncode == 0 and m:
                    ref_wall, ref_steps = float(m.group(1)), int(m.group(2))
                    cpu["reference_backend"] = {"kind": "reference", "what": "genn-team/genn SingleThreadedCPU backend through Runtime::stepTime, generated code built -O3",
                                                "steps": ref_steps, "wall_s": round(ref_wall, 3),
                                                "wall_s_per_sim_s": round(ref_wall / (ref_steps * net.dt / 1000.0), 3), "cores": 1}
                else:
                    cpu["reference_backend"] = {"error": res.stdout[-300:]}
            except Exception as e:      # the baseline is a reported extra: never let it take the bench line down
                cpu["reference_backend"] = {"error": repr(e)}
            finally:
                shutil.rmtree(tmp, ignore_errors=True)

    sim_s = steps * net.dt / 1000.0
    out = {
        "metric": "synaptic_events_per_s", "value": round(events / wall, 1), "unit": "events/s",
        "n_gpus": 1, "steps": steps, "warmup": warmup, "ms_per_step": round(wall / steps * 1e3, 6),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": label, "neurons": num_neurons, "synapses": num_synapses, "dt_ms": net.dt, "seed": net.seed,
                   "stepping": ("resident plan: one launch for all timed steps, state in registers/LDS" if info["resident_plan"] else
                                "hipGraph replay, 100 steps per graph, " + ("1 launch per step" if (info["single_launch_step"] or info["conv_step_in_one_launch"]) else
                                                                           "2 launches per step (synaptic kernels combined)" if (info["combined_synapse_launch"] or info["conv_on_matrix_cores"]) else
                                                                           "2-3 launches per step"))},
        "gsop_per_s": round(events / wall / 1e9, 4),
        "neuron_updates_per_s": round(num_neurons * batch * steps / wall, 1),
        "wall_s_per_sim_s": round(wall / sim_s, 4),
        "events_per_step": round(events / steps, 1), "events_including_warmup": events_with_warmup,
        "algorithmic_gb_per_s_wallclock": round(events * (bytes_per_event or 16) / wall / 1e9, 3),
        "firing_rates_hz": rates,
        "setup_s": {"generate": round(gen_s, 1), "load": round(load_s, 1)},
        "roofline": roofline, "cpu_baseline": cpu,
    }
    if steady is not None:
        out["steady_state"] = steady
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=10000)
    ap.add_argument("--warmup", type=int, default=2000)
    ap.add_argument("--workload", default="potjans")
    ap.add_argument("--cpu-steps", type=int, default=None, help="steps of the CPU baseline sample (default: sized for ~10-20 s)")
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--reference-steps", type=int, default=2000,
                    help="steps of the extra CPU leg on the reference's own SingleThreadedCPU backend (oracle/_ref/ref_driver, "
                         "only where that prebuilt driver exists; 0 disables)")
    ap.add_argument("--profile-steps", type=int, default=2000, help="extra steps replayed with HIP event nodes around every kernel (multiple of 100)")
    ap.add_argument("--steady-steps", type=int, default=10000,
                    help="runs of fewer than 1000 timed steps: steps of the `steady_state` block that follows in the same process (0 disables)")
    ap.add_argument("--steady-warmup", type=int, default=2000, help="untimed steps before the `steady_state` block")
    ap.add_argument("--secondary-steps", type=int, default=1000,
                    help="default workload only: timed steps of the `secondary` block (configuration 3: 10^6 Izhikevich neurons, 10^9 synapses; 0 disables)")
    ap.add_argument("--yardstick-mib", type=int, default=0,
                    help="also run the library's plain copy kernel on this many MiB (5 launches, 2x this traffic each), so a "
                         "hardware-counter run has a kernel of known HBM traffic to scale FETCH_SIZE / WRITE_SIZE by")
    args = ap.parse_args()
    if args.gpus != 1:
        raise SystemExit("bench.py: this build runs on exactly one GPU; --gpus N with N > 1 is not supported "
                         "(the hot path is single-GPU: sharded by postsynaptic neuron it would exchange only the spike lists each step)")

    if args.workload == "init_izhikevich":
        return bench_init(args)
    if args.workload in ("izh_procedural", "izh_stored"):
        print(json.dumps(bench_procedural(args, stored=(args.workload == "izh_stored"))))
        return

    out = run_net_workload(args, args.workload, args.steps, args.warmup, args.profile_steps, with_cpu=not args.no_cpu, with_steady=True)
    if args.workload == "potjans" and args.secondary_steps > 0:
        # configuration 3 as it stands (the bandwidth-bound case), generated on the host and uploaded like the headline network
        try:
            sec = run_net_workload(args, "izh", args.secondary_steps, 100, min(args.secondary_steps, 1000), with_cpu=False, with_steady=False)
            out["secondary"] = {k: sec[k] for k in ("metric", "value", "unit", "steps", "warmup", "ms_per_step", "dtype", "data", "config", "gsop_per_s",
                                                    "neuron_updates_per_s", "wall_s_per_sim_s", "events_per_step", "firing_rates_hz", "setup_s", "roofline")}
        except Exception as e:          # a reported extra: never let it take the bench line down
            out["secondary"] = {"error": repr(e)}
    print(json.dumps(out))


if __name__ == "__main__":
    main()
