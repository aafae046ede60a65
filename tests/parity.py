"""Shared driver for the GPU parity tests: run a Net on the MI355X engine and on the CPU oracle
side by side and compare with the bars the hot path is held to:
spike queues bit-exact every step, state within 1e-5 relative (bit-exact where no fp32 sum can
be reordered)."""
import numpy as np

from genn_amd.genn_model import model_from_net
from oracle.genn_cpu import OracleNet

REL_TOL = 1e-5


def assert_close(got, want, what, exact, accumulator=False):
    """``accumulator``: the array holds sums of mixed-sign weights added by atomics.  A reordered
    fp32 sum errs by ulps of its partial sums, not of its (possibly cancelled) result, so such
    arrays are held to 1e-5 of the larger of the element and the array's peak magnitude."""
    if exact:
        assert np.array_equal(got, want), f"{what}: {np.count_nonzero(got != want)} of {got.size} elements differ"
    else:
        floor = max(1e-3, float(np.abs(want).max(initial=0.0))) if accumulator else 1e-3
        scale = np.maximum(np.abs(want), floor)
        err = np.abs(got.astype(np.float64) - want.astype(np.float64)) / scale
        assert err.max(initial=0.0) <= REL_TOL, f"{what}: max relative error {err.max():.3e}"


def run_side_by_side(net, steps=None, check_every=1, exact=True, use_graph=False, span=None, exact_steps=None):
    """Returns (model, oracle, spike counts per population).  ``exact_steps``: number of leading steps
    over which rasters must be identical even when ``exact`` is False (then later steps only
    compare while the two rasters still agree)."""
    steps = steps or net.steps
    model = model_from_net(net, span=span)
    model.load(num_recording_timesteps=steps)
    oracle = OracleNet(net, num_recording_timesteps=steps,
                       col_stride={s.name: model.synapse_populations[s.name].col_stride for s in net.syns if s.wum in ("stdp_trace", "stdp_additive")} or None)
    counts = {p.name: 0 for p in net.pops}
    diverged = False
    for step in range(steps):
        if use_graph and step % check_every == 0 and step + check_every <= steps:
            pass
        model.step_time()
        oracle.step()
        for p in net.pops:
            got = model.neuron_populations[p.name].current_spikes[0]
            want = oracle.spikes(p.name)
            counts[p.name] += len(want)
            if exact or (exact_steps is not None and step < exact_steps):
                assert np.array_equal(got, want), f"step {step}: spike queue of {p.name} differs ({len(got)} vs {len(want)})"
            elif not np.array_equal(got, want):
                diverged = True
        if diverged:
            break
        if (step + 1) % check_every == 0:
            compare_state(net, model, oracle, f"step {step}", exact)
    return model, oracle, counts


def compare_state(net, model, oracle, where, exact):
    for p in net.pops:
        g = model.neuron_populations[p.name]
        if p.model == "ssa":
            assert np.array_equal(g.vars["startSpike"].pull_from_device(), oracle.start_spike(p.name)), f"{where}: startSpike of {p.name}"
            continue
        names = ("V", "RefracTime") if p.model == "lif" else ("V", "U")
        for k, name in enumerate(names):
            assert_close(g.vars[name].pull_from_device(), oracle.var(p.name, k), f"{where}: {name} of {p.name}", exact)
    for s in net.syns:
        sg = model.synapse_populations[s.name]
        if sg.fused_ps_target is sg:
            assert_close(sg.vars["outPost"].pull_from_device(), oracle.out_post(s.name), f"{where}: outPost of {s.name}", exact, accumulator=True)
            if "denDelay" in sg.vars:
                got, want = sg.vars["denDelay"].pull_from_device().copy(), oracle.den_delay(s.name).copy()
                if model.runner_info()["single_launch_step"]:
                    # zero-delay synapses of the last step's spikes already sit in the slot that will be read next
                    # (the reference adds them at the start of the next step): leave that slot out here; the
                    # neuron state compared above depends on every slot's total
                    D, n = s.max_den_delay, net.pop(s.trg).n
                    nxt = (model.timestep + 1) % D
                    got.reshape(D, n)[nxt] = 0
                    want.reshape(D, n)[nxt] = 0
                assert_close(got, want, f"{where}: denDelay of {s.name}", exact, accumulator=True)
        if s.wum == "stdp_additive":
            assert_close(sg.vars["g"].pull_from_device(), oracle.syn_g(s.name), f"{where}: g of {s.name}", exact)
        if s.wum == "stdp_trace":
            assert_close(sg.vars["g"].pull_from_device(), oracle.syn_g(s.name), f"{where}: g of {s.name}", exact)
            assert_close(sg.vars["preTrace"].pull_from_device(), oracle.pre_trace(s.src), f"{where}: preTrace of {s.name}", exact)
            assert_close(sg.vars["postTrace"].pull_from_device(), oracle.post_trace(s.trg), f"{where}: postTrace of {s.name}", exact)
