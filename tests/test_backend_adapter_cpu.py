"""Code generation through the GeNN backend adapter, without a GPU: the reference's generator, given
`GeNN::CodeGenerator::MI355X::Backend`, must produce a runner that compiles with the host compiler alone and
exports exactly the entry points Runtime binds (runtime.cc:87-94, generateRunner.cc:308-321) plus one
pushMerged<Name>Group<i>ToDevice per merged group."""
import os
import shutil
import subprocess
import sys
import tempfile

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
sys.path.insert(0, os.path.join(HERE, "golden"))

from cases import CASES  # noqa: E402
from genn_amd.netspec import write_netspec  # noqa: E402

DRIVER = os.path.join(ROOT, "oracle", "_ref", "mi355x_driver")
pytestmark = pytest.mark.skipif(not os.path.exists(DRIVER), reason="oracle/_ref/mi355x_driver is not built (needs the reference tree at build time)")


def _generate(case):
    net, snap = CASES[case]()
    net.snap = snap
    tmp = tempfile.mkdtemp(prefix="adapter_gen_")
    spec, work, out = (os.path.join(tmp, d) for d in ("spec", "work", "out"))
    for d in (work, out):
        os.makedirs(d)
    write_netspec(net, spec)
    res = subprocess.run([DRIVER, spec, work, out, "--generate-only"], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=300)
    assert res.returncode == 0, res.stdout[-3000:]
    code = os.path.join(work, net.name + "_CODE")
    return net, tmp, code


def _exports(lib):
    out = subprocess.run(["nm", "-D", "--defined-only", lib], stdout=subprocess.PIPE, text=True, check=True).stdout
    return {line.split()[-1] for line in out.splitlines() if " T " in line}


@pytest.mark.parametrize("case", ["stdp_small", "stdp_additive_small", "potjans_small", "conv_small", "dense_small", "va_delay_small", "graded_small", "reverse_small"])
def test_generated_runner_exports_reference_entry_points(case):
    net, tmp, code = _generate(case)
    try:
        exports = _exports(os.path.join(code, "librunner.so"))
        for name in ("allocateMem", "freeMem", "initialize", "initializeSparse", "initializeHost", "stepTime", "updateNeurons", "updateSynapses"):
            assert name in exports, f"{name} missing from the generated runner"
        pushes = {e for e in exports if e.startswith("pushMerged")}
        assert any(e.startswith("pushMergedNeuronUpdateGroup") for e in pushes)
        assert any(e.startswith("pushMergedPresynapticUpdateGroup") for e in pushes)
        if case in ("stdp_small", "stdp_additive_small"):
            assert any(e.startswith("pushMergedPostsynapticUpdateGroup") for e in pushes)
            assert "pushMergedNeuronUpdate0spikeTimesToDevice" in exports or any("spikeTimes" in e for e in pushes)
        if case == "stdp_additive_small":
            synapse_code = open(os.path.join(code, "synapseUpdate.cc")).read()
            assert "d.wum = 6u" in synapse_code and "d.tauMinus = v[g]" in synapse_code and "d.tauPlus = v[g]" in synapse_code and "d.preTrace" not in synapse_code
        # the runner is host code: no device code object, only a link against the device library
        ldd = subprocess.run(["ldd", os.path.join(code, "librunner.so")], stdout=subprocess.PIPE, text=True).stdout
        assert "libgenn_mi355x.so" in ldd
        neuron = open(os.path.join(code, "neuronUpdate.cc")).read()
        assert "gennmi_push_neuron_update_group" in neuron and "gennmi_step" in neuron and "__global__" not in neuron
        synapse = open(os.path.join(code, "synapseUpdate.cc")).read()
        assert synapse.count("gennmi_push_presynaptic_update_group") >= 1
        if case == "potjans_small":
            assert "d.maxDenDelay" in synapse and "d.denDelay" in synapse
        if case == "conv_small":
            assert "d.conv[7]" in synapse
        init = open(os.path.join(code, "init.cc")).read()
        assert "gennmi_push_mirrors" in init
        if case in ("stdp_small", "stdp_additive_small"):
            assert "gennmi_build_remap" in init
    finally:
        shutil.rmtree(tmp, ignore_errors=True)


def test_procedural_projections_generate():
    """PROCEDURAL matrices through the adapter: the built-in connectivity and weight snippets are recognised by identity and
    become the descriptor's `procedural` block (seed, snippet, streams 2k + 1 / 2k + 2 by projection name, parameters)."""
    from genn_amd import configs
    net = configs.procedural()
    net.snap = 50
    tmp = tempfile.mkdtemp(prefix="adapter_proc_")
    try:
        spec, work, out = (os.path.join(tmp, d) for d in ("spec", "work", "out"))
        for d in (work, out):
            os.makedirs(d)
        write_netspec(net, spec)
        res = subprocess.run([DRIVER, spec, work, out, "--generate-only"], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=300)
        assert res.returncode == 0, res.stdout[-3000:]
        code = open(os.path.join(work, net.name + "_CODE", "synapseUpdate.cc")).read()
        assert code.count("d.procedural.seed = 31ull") == 4
        for streams in ("a[] = {1u}, b[] = {2u}", "a[] = {3u}, b[] = {4u}", "a[] = {5u}, b[] = {6u}", "a[] = {7u}, b[] = {8u}"):
            assert streams in code
        assert "d.rowLength" not in code and "d.ind" not in code           # nothing stored, nothing bound
    finally:
        shutil.rmtree(tmp, ignore_errors=True)


def test_poisson_sources_generate():
    """PoissonExp current sources through the adapter: recognised by their injection code (currentSourceModels.h:107-122), they
    become descriptors with the model's seed, one generator stream per source (1000 + its place in the name-ordered list
    of the model's current sources) and the snippet's derived parameters; the runner stays host code."""
    from genn_amd import configs
    net = configs.potjans(neuron_scale=0.02, connectivity_scale=0.2, steps=10, poisson=True)
    net.snap = 10
    tmp = tempfile.mkdtemp(prefix="adapter_poisson_")
    try:
        spec, work, out = (os.path.join(tmp, d) for d in ("spec", "work", "out"))
        for d in (work, out):
            os.makedirs(d)
        write_netspec(net, spec)
        res = subprocess.run([DRIVER, spec, work, out, "--generate-only"], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=300)
        assert res.returncode == 0, res.stdout[-3000:]
        code = open(os.path.join(work, net.name + "_CODE", "neuronUpdate.cc")).read()
        assert f"d.cs[0].kind = 2u" in code and "d.cs[0].seed = 4321ull" in code
        assert "{1000u, 1001u, 1002u, 1003u, 1004u, 1005u, 1006u, 1007u}; d.cs[0].stream = v[g]" in code
        for field in ("init", "expDecay", "expMinusLambda", "current"):
            assert f"d.cs[0].{field} = " in code
        assert "gennrand" not in code and "__global__" not in code
    finally:
        shutil.rmtree(tmp, ignore_errors=True)


@pytest.mark.parametrize("dynamic, case", [("neuron:E.Ioffset", "va_small"), ("ps:EE.tau", "va_small"), ("cs:23E_dc.amp", "potjans_small"),
                                           ("wu:EE.aPlus", "stdp_small")])
def test_dynamic_parameters_are_refused(dynamic, case):
    """The device library's descriptors hold parameters as constants built before the first step, so with the library's
    kernels asked for explicitly a model that marks a parameter dynamic (setParamDynamic; the reference gives it a DYNAMIC
    merged-struct field, neuronGroup.h:135, currentSource.h:67, synapseGroup.h:187-190) must be refused at generation
    time instead of running with the value frozen.  (Left to choose, the backend generates kernels for such a model.)"""
    net, snap = CASES[case]()
    net.snap = snap
    tmp = tempfile.mkdtemp(prefix="adapter_dyn_")
    try:
        spec, work, out = (os.path.join(tmp, d) for d in ("spec", "work", "out"))
        for d in (work, out):
            os.makedirs(d)
        write_netspec(net, spec)
        res = subprocess.run([DRIVER, spec, work, out, "--generate-only", "--kernels=library", "--dynamic=" + dynamic], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=300)
        assert res.returncode != 0
        assert "dynamic" in res.stdout and dynamic.split(".")[-1] in res.stdout and "not among the models" in res.stdout, res.stdout[-2000:]
    finally:
        shutil.rmtree(tmp, ignore_errors=True)


def _assert_host_passes_hold_no_hip(code):
    """What the host compiler sees of a generated runner — every module outside its `#ifdef __HIPCC__` section — holds no
    launch syntax, no HIP call and no HIP header: device code is reached through the device library's C ABI only.  The
    objects were in fact built that way: the host pass is $(CXX), the device pass `hipcc --genco`."""
    import re
    for name in sorted(os.listdir(code)):
        if not name.endswith((".cc", ".h")):
            continue
        text = open(os.path.join(code, name)).read()
        host = re.sub(r"#ifdef __HIPCC__.*?(#else|#endif)", "", text, flags=re.S)
        assert "<<<" not in host, name
        assert not re.search(r"\bhip[A-Z]\w*\s*\(", host), (name, re.search(r"\bhip[A-Z]\w*\s*\(", host))
        assert "hip_runtime" not in host, name
    makefile = open(os.path.join(code, "Makefile")).read()
    assert "$(CXX) $(CXXFLAGS) -MF" in makefile and "$(HIPCC) $(HIPCCFLAGS)" in makefile and "CXX :=" not in makefile
    undefined = subprocess.run(["nm", "-D", "--undefined-only", os.path.join(code, "librunner.so")], stdout=subprocess.PIPE, text=True, check=True).stdout
    assert "gennmi_program_update" in undefined and not re.search(r"\bhip[A-Z]", undefined), undefined


def _generate_with(case, *options):
    if case == "procedural":        # (no fixture: nothing in the reference's CPU backend regenerates matrices)
        from genn_amd import configs
        net, snap = configs.procedural(), 50
    else:
        net, snap = CASES[case]()
    net.snap = snap
    tmp = tempfile.mkdtemp(prefix="adapter_genk_")
    spec, work, out = (os.path.join(tmp, d) for d in ("spec", "work", "out"))
    for d in (work, out):
        os.makedirs(d)
    write_netspec(net, spec)
    res = subprocess.run([DRIVER, spec, work, out, "--generate-only", *options], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=300)
    return net, tmp, os.path.join(work, net.name + "_CODE"), res


@pytest.mark.parametrize("case, options", [("custom_update_small", ("--kernels=generated",)), ("va_double_small", ()), ("post_events_small", ()), ("custom_small", ()), ("dynamic_small", ()), ("poisson_input_small", ()), ("synapse_dynamics_small", ()), ("prev_times_small", ()), ("stdp_delay_small", ()), ("graded_small", ("--kernels=generated",)), ("conv_small", ("--kernels=generated",)), ("procedural", ("--kernels=generated",)), ("dense_small", ("--kernels=generated",)), ("stdp_small", ("--kernels=generated",)),
                                           ("va_small", ("--dynamic=neuron:E.Ioffset",)), ("potjans_small", ("--kernels=generated",))])
def test_generated_kernels_are_chosen_and_build(case, options):
    """Models of the driver's own, dynamic parameters, or Preferences::kernelSource = GENERATED: the modules then hold device
    code (the model's snippets inside this backend's kernel skeletons), built into gfx950 code objects by the runner's own
    Makefile and embedded in the modules' objects; the runner itself is host C++ that launches them through the device
    library's C ABI, with the reference's entry points around it."""
    net, tmp, code, res = _generate_with(case, *options)
    try:
        assert res.returncode == 0, res.stdout[-3000:]
        neuron = open(os.path.join(code, "neuronUpdate.cc")).read()
        synapse = open(os.path.join(code, "synapseUpdate.cc")).read()
        assert "__global__" in neuron and "gennmi_kernel::orderedSlot" in neuron and "gennmi_kernel::recordBallot" in neuron
        assert "__global__" in synapse and "gennmi_kernel::addScalar" in synapse
        assert "gennmi_runner_create" not in open(os.path.join(code, "runner.cc")).read()
        makefile = open(os.path.join(code, "Makefile")).read()
        assert "hipcc" in makefile and "--genco" in makefile and "--offload-arch=gfx950" in makefile and "-packed-fp32-ops" in makefile and "-ffp-contract=off" in makefile
        _assert_host_passes_hold_no_hip(code)
        # a bounded wait of the spike compaction that expires raises the program's error flag, whatever the timing setting:
        # the kernels get the flag from the library, which reports it from the next call that waits for the device
        assert "a.error = gennmiProgramError" in neuron and "gennmi_program_error_flag(gennmiProgram, &gennmiProgramError)" in open(os.path.join(code, "runner.cc")).read()
        assert "gennmiError, gennmiLaunch.spinLimit)" in neuron
        exports = _exports(os.path.join(code, "librunner.so"))
        for name in ("allocateMem", "freeMem", "initialize", "initializeSparse", "stepTime", "updateNeurons", "updateSynapses"):
            assert name in exports
        if case == "custom_update_small":
            # custom updates: one entry point per update group under the reference's name, its kernels generated from the
            # update code
            custom = open(os.path.join(code, "customUpdate.cc")).read()
            for group in ("Homeostasis", "Decay", "Reduce"):
                assert "update" + group in exports
            assert "gennmi_program_launch(gennmiProgram, gennmiCustomUpdateHomeostasisKernelId" in custom and "gennmi_program_launch(gennmiProgram, gennmiCustomUpdateWUDecayKernelId" in custom
            # (order within a group as in the reference: per-neuron, per-synapse, transpose)
            assert custom.index("gennmi_program_launch(gennmiProgram, gennmiCustomUpdateWUDecayKernelId") < custom.index("gennmi_program_launch(gennmiProgram, gennmiCustomUpdateTransposeDecayKernelId")
            assert "gennmi_kernel::blockReduceSum(_lrsum)" in custom and "gennmi_kernel::blockReduceMax(_lrpeak)" in custom
            assert "gennmi_kernel::groupOfBlock(gennmiCustomUpdateWUDecayStarts" in custom
            assert "group->variableTranspose[" in custom and "gennmiTile[tx][ty + j]" in custom
            assert "if(col < group->rowLength[row])" in custom
            assert "gennmiUploadCustomUpdateGroups();" in open(os.path.join(code, "runner.cc")).read()
        if case == "potjans_small":
            # dendritic delay: the neuron update's last work-group moves the ring pointers on; it is found by a count in two
            # levels (sixteen work-groups to a word, a cache line per word), not by every work-group adding to one word
            assert "gennmiLastToFinish = last;" in neuron and "gennmiArgs.finished + 32u * (1u + group)" in neuron
            assert "* sizeof(uint32_t)));" in neuron and "GENNMI_CHECK(gennmi_malloc(&p, sizeof(uint32_t)));" not in neuron
            # the presynaptic walk asks for an item's queue entry one item ahead
            assert "idPreNext = group->srcSpk[" in synapse and "const unsigned int idPre = idPreNext;" in synapse
        if case == "custom_small":
            # the extra state variable and the weight-update variables are in the kernels under the reference's names
            assert "group->A[id]" in neuron and "sPreOutSynWUMPre" in neuron and "sPostInSynWUMPost" in neuron
            assert "group->wPost[idSyn] = group->sPost[idPost]" in synapse and "group->wPre[rowMajorIndex] = group->sPre[idPre]" in synapse
        if case == "va_double_small":
            # a double-precision model takes generated kernels by itself (the library's are fp32): state and accumulators are fp64
            assert "double* __restrict__ V" in neuron.replace("double * ", "double* ") and "gennmi_kernel::addScalar(&group->outPost" in synapse
            assert "double t" in neuron or "float t" in neuron
        if case == "post_events_small":
            # spike-like events of the postsynaptic population: queued by the neuron update like presynaptic ones, walked through
            # the column view before the true spikes
            assert "trgSpkCntEvent" in synapse and "trgSpkEvent" in synapse and "group->hits[rowMajorIndex]" in synapse
            assert "gennmiEvent0 = true" in neuron
        if case == "procedural":
            # PROCEDURAL connectivity and weights: the snippets' own code inside the presynaptic walk, drawing from a generator
            # keyed by (seed, projection, row, lane) at step 0
            assert "gennmi_kernel::rngBegin(gennmiSeed, (1u), (unsigned long long)idPre * 1u + j, 0ull)" in synapse
            assert "gennmi_kernel::rngUniform(gennmiRng)" in synapse and "gennmi_kernel::rngNormal(gennmiRng)" in synapse
            assert "const unsigned int idPost = " in synapse and "_prevJ" in synapse
        if case == "conv_small":
            # TOEPLITZ connectivity: the snippet's diagonal build code inside the presynaptic walk, its addSynapse become the update
            assert "const unsigned int idPost = " in synapse and "idKernel0" in synapse and "idKernel3" in synapse
        if case == "prev_times_small":
            # previous spike times: a kernel of its own stamps last step's spikes before the update
            assert neuron.index('gennmiProgram, module, "gennmiPrevSpikeTimeKernel"') < neuron.index('gennmiProgram, module, "gennmiNeuronUpdateKernel"')
            assert "group->prevST[" in neuron
        if case == "graded_small":
            # spike-like events: a queue per condition, compacted in order like the true spikes and recorded from the ballot
            assert "gennmiEvent0 = true" in neuron and "eventSlot0 = gennmi_kernel::orderedSlot(gennmiEvent0" in neuron and "recordSpkEvent" in neuron
            assert "srcSpkCntEvent" in synapse or "srcSpkCntEvent".lower() in synapse.lower()
        if case == "stdp_delay_small":
            # a learning rule over delay slots: chosen for generated kernels by itself; the populations' ring pointers move on
            # in a kernel of their own before the update, and the queues are read through GeNN's delay-slot helpers
            assert neuron.index('gennmiProgram, module, "gennmiSpikeQueueUpdateKernel"') < neuron.index('gennmiProgram, module, "gennmiNeuronUpdateKernel"')
            assert "writeDelaySlot" in neuron and "preDelaySlot" in synapse
        if case == "synapse_dynamics_small":
            # code that runs for every synapse every step: a kernel of its own, launched before the presynaptic update
            assert synapse.index('gennmiProgram, module, "gennmiSynapseDynamicsKernel"') < synapse.index('gennmiProgram, module, "gennmiPresynapticUpdateKernel"')
            assert "group->x[idSyn]" in synapse and "group->Vpre[row]" in synapse
        if case == "poisson_input_small":
            # gennrand_exponential() of the built-in Poisson neuron: a counter-based generator keyed by the model's seed, one
            # stream per population, the step counted by the launcher
            assert "gennmi_kernel::rngBegin(gennmiSeed, (2000u), id, gennmiStep)" in neuron and "gennmi_kernel::rngExponential(gennmiRng)" in neuron
            assert f"a.seed = {net.seed}ull;" in neuron and "const unsigned long long gennmiStep = gennmiEntry.step;" in neuron
        if case in ("dynamic_small", "va_small"):
            # the dynamic parameter is a struct field the kernel reads, with a push function that marks the device copy stale
            assert "group->Ioffset" in neuron
            assert any(e.startswith("pushMergedNeuronUpdate") and e.endswith("IoffsetToDevice") for e in exports)
            assert "gennmiStructsDirty = true" in open(os.path.join(code, "runner.cc")).read()
    finally:
        shutil.rmtree(tmp, ignore_errors=True)


def test_generated_kernels_take_the_batch_from_the_grid():
    """A batched model on generated kernels: the launches have the batch as the grid's second dimension and the kernels
    index neuron variables, spike queues, recording words and per-synapse variables by it (GeNN's own index helpers)."""
    import numpy as np
    net, snap = CASES["custom_small"]()
    net.snap = snap
    net.batch_size = 2
    for p in net.pops:
        p.vars = {v: np.stack([a, a]) for v, a in p.vars.items()}
    tmp = tempfile.mkdtemp(prefix="adapter_genk_batch_")
    try:
        spec, work, out = (os.path.join(tmp, d) for d in ("spec", "work", "out"))
        for d in (work, out):
            os.makedirs(d)
        write_netspec(net, spec)
        res = subprocess.run([DRIVER, spec, work, out, "--generate-only"], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=300)
        assert res.returncode == 0, res.stdout[-3000:]
        code = os.path.join(work, net.name + "_CODE")
        neuron = open(os.path.join(code, "neuronUpdate.cc")).read()
        synapse = open(os.path.join(code, "synapseUpdate.cc")).read()
        assert "u, 2u, 256u, &a, sizeof(a)" in neuron and "u, 2u, 256u, &a, sizeof(a)" in synapse
        assert "group->A[batchOffset + id]" in neuron and "[blockIdx.y] = slot.total" in neuron
        assert "(size_t)recordingTimestep * 2u + blockIdx.y" in neuron
        assert "group->srcSpk[preBatchOffset + spikeNext]" in synapse and "group->wPost[synBatchOffset + idSyn]" in synapse
    finally:
        shutil.rmtree(tmp, ignore_errors=True)


def test_custom_updates_take_the_batch_from_the_grid_and_reduce_over_it():
    """Custom updates of a batched model: per-batch updates read the batch from the grid's second dimension, a reduction over
    batches loops over them in the lane that owns the element, and the device library's own kernels refuse a model with custom
    updates by name (their kernels are generated)."""
    net, snap = CASES["custom_update_small"]()
    net.snap = snap
    net.batch_size = 3
    tmp = tempfile.mkdtemp(prefix="adapter_custom_batch_")
    try:
        spec, work, out = (os.path.join(tmp, d) for d in ("spec", "work", "out"))
        for d in (work, out):
            os.makedirs(d)
        write_netspec(net, spec)
        res = subprocess.run([DRIVER, spec, work, out, "--generate-only"], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=300)
        assert res.returncode == 0, res.stdout[-3000:]
        custom = open(os.path.join(work, net.name + "_CODE", "customUpdate.cc")).read()
        assert "gennmi_program_launch(gennmiProgram, " in custom and "u, 3u, 256u, &a, sizeof(a)" in custom
        assert "for(unsigned int batch = 0; batch < 3u; batch++)" in custom
        # the per-neuron update and the reduction over neurons run once per batch, the static dense weights once
        assert "group->applied[batchOffset + id]" in custom and "group->sum[blockIdx.y] = _lrsum" in custom
        assert "if(blockIdx.y == 0u && id < size)" in custom
    finally:
        shutil.rmtree(tmp, ignore_errors=True)


def test_custom_updates_beside_library_kernels():
    """A model of built-in snippets with custom updates keeps the device library's kernels for its step (descriptors, no
    device code in neuronUpdate.cc) and gets generated kernels for the custom updates only: queued steps are flushed before
    they launch, and the arrays they may have written are named to the library, which refreshes what it derives from them."""
    net, tmp, code, res = _generate_with("custom_update_small")
    try:
        assert res.returncode == 0, res.stdout[-3000:]
        neuron = open(os.path.join(code, "neuronUpdate.cc")).read()
        custom = open(os.path.join(code, "customUpdate.cc")).read()
        runner = open(os.path.join(code, "runner.cc")).read()
        assert "__global__" not in neuron and "gennmi_push_neuron_update_group" in neuron and "gennmi_runner_create" in runner
        assert "__global__" in custom and "gennmi_program_launch(gennmiProgram, gennmiCustomUpdateWUDecayKernelId" in custom
        body = custom[custom.index("void updateDecay("):]
        assert body.index("gennmi_program_launch(") < body.index("gennmi_note_mirror_write(")
        # written: the weights both decays refer to and the transpose target; the read-only reference of the reduction is not
        assert "gennmi_note_mirror_write(mergedCustomUpdateTransposeWUGroup0[g].variableTranspose)" in custom
        reduce = custom[custom.index("void updateReduce("):]
        assert "gennmi_note_mirror_write" not in reduce[:reduce.index("\n}")]
        assert "gennmiUploadCustomUpdateGroups();" in runner
        assert "hipcc" in open(os.path.join(code, "Makefile")).read()
        exports = _exports(os.path.join(code, "librunner.so"))
        for name in ("updateHomeostasis", "updateDecay", "updateReduce", "stepTime"):
            assert name in exports
    finally:
        shutil.rmtree(tmp, ignore_errors=True)


def test_custom_connectivity_updates_generate_and_build():
    """Custom connectivity updates: a lane per row runs the row update code (add_synapse / remove_synapse and the bookkeeping
    of every variable on the synapses are GeNN's), the column view of a projection that learns from postsynaptic spikes is
    rebuilt by the device library afterwards, and the model takes generated kernels by itself; asked for the library's step
    kernels, the backend says why not."""
    net, tmp, code, res = _generate_with("rewiring_small")
    try:
        assert res.returncode == 0, res.stdout[-3000:]
        assert "__global__" in open(os.path.join(code, "neuronUpdate.cc")).read()
        custom = open(os.path.join(code, "customUpdate.cc")).read()
        assert "gennmi_program_launch(gennmiProgram, gennmiCustomConnectivityUpdatePruneKernelId" in custom and "gennmi_program_launch(gennmiProgram, gennmiCustomConnectivityUpdateSproutKernelId" in custom
        prune = custom[custom.index("void updatePrune("):]
        assert prune.index("gennmi_program_launch(gennmiProgram, gennmiCustomConnectivityUpdatePruneKernelId") < prune.index("gennmi_build_remap(")
        # host update code first: plain host code over the host buffers, pushed to the device buffers behind them
        assert "group->limit[_i] = " in prune and prune.index("gennmi_memcpy_to_device(gennmiDev(group->limit), group->limit") < prune.index("gennmi_program_launch(")
        # the removed synapse's slot takes the row's last one, with the weight and the other custom updates' variables
        assert "group->ind[idx] = group->ind[lastIdx];" in custom and "group->dependentVar0[idx] = group->dependentVar0[lastIdx];" in custom
        assert "group->rowLength[id]--;" in custom and "group->rowLength[id]++;" in custom
        exports = _exports(os.path.join(code, "librunner.so"))
        assert "updatePrune" in exports and "updateSprout" in exports and "updateDecay" in exports
    finally:
        shutil.rmtree(tmp, ignore_errors=True)
    net, tmp, code, res = _generate_with("rewiring_small", "--kernels=library")
    try:
        assert res.returncode != 0 and "custom connectivity updates beside the device library's step kernels" in res.stdout, res.stdout[-2000:]
    finally:
        shutil.rmtree(tmp, ignore_errors=True)


def test_narrow_sparse_indices_take_generated_kernels():
    """ModelSpec::setDefaultNarrowSparseIndEnabled stores the targets of SPARSE rows in the narrowest type that holds them; the device
    library reads 32-bit targets, so such a model takes generated kernels, whose code takes the type from the merged struct."""
    net, tmp, code, res = _generate_with("va_small", "--narrow-ind")
    try:
        assert res.returncode == 0, res.stdout[-3000:]
        synapse = open(os.path.join(code, "synapseUpdate.cc")).read()
        assert "__global__" in synapse and "uint16_t* __restrict__ ind" in synapse.replace("uint16_t * ", "uint16_t* ")
    finally:
        shutil.rmtree(tmp, ignore_errors=True)


def test_library_kernels_say_what_they_do_not_cover():
    """Asked for the device library's own kernels for something they do not cover (a double-precision model: they are fp32), the
    backend says so."""
    net, snap = CASES["va_small"]()
    net.snap = snap
    tmp = tempfile.mkdtemp(prefix="adapter_genk_refuse_")
    try:
        spec, work, out = (os.path.join(tmp, d) for d in ("spec", "work", "out"))
        for d in (work, out):
            os.makedirs(d)
        write_netspec(net, spec)
        res = subprocess.run([DRIVER, spec, work, out, "--generate-only", "--kernels=library", "--precision=double"], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=300)
        assert res.returncode != 0
        assert "single-precision" in res.stdout, res.stdout[-2000:]
    finally:
        shutil.rmtree(tmp, ignore_errors=True)


def test_device_initialisation_is_generated_on_request():
    """Preferences::deviceInitialisation: built-in connectivity and per-synapse variable snippets of SPARSE projections become
    calls of the device library's generators (with the model's seed and one stream per array), each followed by a note that
    the device now holds the array (so that the upload which ends initialize() leaves it alone); host code that walks rows asks
    for the copy first; without the switch the reference's generic initialisation code runs on the host as before."""
    from genn_amd import configs
    net = configs.snippet_initialised(n_e=200, n_i=50, steps=10)
    net.snap = 0
    layers = configs.snippet_initialised_layers(steps=10)
    layers.snap = 0
    tmp = tempfile.mkdtemp(prefix="adapter_devinit_")
    try:
        spec = os.path.join(tmp, "spec")
        write_netspec(net, spec)
        for flag in (True, False):
            work, out = os.path.join(tmp, f"work{int(flag)}"), os.path.join(tmp, f"out{int(flag)}")
            os.makedirs(work); os.makedirs(out)
            res = subprocess.run([DRIVER, spec, work, out, "--generate-only"] + (["--device-init"] if flag else []),
                                 stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=300)
            assert res.returncode == 0, res.stdout[-3000:]
            init = open(os.path.join(work, net.name + "_CODE", "init.cc")).read()
            assert ("gennmi_init_sparse_fixed_probability(" in init) == flag
            assert ("gennmi_init_sparse_fixed_number_post(" in init) == flag
            assert ("gennmi_init_var(" in init) == flag
            assert "gennmi_mirrors_begin_initialisation()" in init
            if flag:
                assert f"{net.seed}ull" in init and "gennmi_memcpy_from_device(" not in init
                assert init.count("gennmi_mirror_device_initialised(") >= 8 and "gennmi_mirror_ensure_host(" not in init
                # EI has a constant weight (no variable), so three weight arrays are drawn; four matrices are generated
                assert init.count("gennmi_init_var(") == 3 or init.count("gennmi_init_var(") == 2
        # Conv2D with kernel-initialised weights and FixedNumberPreWithReplacement
        spec = os.path.join(tmp, "spec_layers")
        write_netspec(layers, spec)
        for flag in (True, False):
            work, out = os.path.join(tmp, f"work_layers{int(flag)}"), os.path.join(tmp, f"out_layers{int(flag)}")
            os.makedirs(work); os.makedirs(out)
            res = subprocess.run([DRIVER, spec, work, out, "--generate-only"] + (["--device-init", "--device-arrays"] if flag else []),
                                 stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=300)
            assert res.returncode == 0, res.stdout[-3000:]
            init = open(os.path.join(work, layers.name + "_CODE", "init.cc")).read()
            assert ("gennmi_init_sparse_fixed_number_pre(" in init) == flag
            # (connectivity, then once more per kernel-initialised variable)
            assert init.count("gennmi_init_sparse_conv2d(") == (2 if flag else 0)
            if not flag:
                assert "idKernel0" in init and "idKernel3" in init
    finally:
        shutil.rmtree(tmp, ignore_errors=True)


def test_profiler_ranges_are_generated_on_request():
    """Preferences::profilerRanges (the CUDA backend's enableNVTX, cuda/backend.cc:741-752): stepTime, updateSynapses and
    updateNeurons are bracketed by gennmi_profiler_range_push / _pop in the generated runner (generateRunner.cc:275-297), and
    not otherwise."""
    from cases import CASES
    net, snap = CASES["va_small"]()
    net.snap = snap
    tmp = tempfile.mkdtemp(prefix="adapter_ranges_")
    try:
        spec = os.path.join(tmp, "spec")
        write_netspec(net, spec)
        for flag in (True, False):
            work, out = os.path.join(tmp, f"work{int(flag)}"), os.path.join(tmp, f"out{int(flag)}")
            os.makedirs(work); os.makedirs(out)
            res = subprocess.run([DRIVER, spec, work, out, "--generate-only"] + (["--profiler-ranges"] if flag else []),
                                 stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=300)
            assert res.returncode == 0, res.stdout[-3000:]
            runner = open(os.path.join(work, net.name + "_CODE", "runner.cc")).read()
            for name in ("stepTime", "updateSynapses", "updateNeurons"):
                assert (f'gennmi_profiler_range_push("{name}");' in runner) == flag
            assert runner.count("gennmi_profiler_range_pop();") == (3 if flag else 0)
    finally:
        shutil.rmtree(tmp, ignore_errors=True)
