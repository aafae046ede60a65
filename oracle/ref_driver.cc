// Test infrastructure, not product code.
//
// Drives the reference's OWN SingleThreadedCPU backend (built by oracle/Makefile.ref into
// oracle/_ref/) on a network described by a "netspec" directory written by
// genn_amd/netspec.py, and dumps spike rasters and state snapshots.  Those dumps become the
// golden fixtures under tests/golden/ and validate the C restatement in oracle/genn_cpu.c.
//
// The flow follows the reference's generator driver (src/genn/generator/generator.cc:55-121):
// ModelSpecInternal -> finalise -> createBackend -> ModelSpecMerged -> generateAll ->
// generateMakefile -> make -> Runtime -> allocate / initialize / (load arrays) /
// initializeSparse / stepTime.  All inputs (connectivity, weights, delays, initial state,
// spike-source arrays, noise) are LOADED from the netspec; none of the reference's seeded
// initialisation snippets is used, because their draw order cannot be reproduced elsewhere.
//
// usage: ref_driver <netspec dir> <work dir> <out dir>
#include <algorithm>
#include <chrono>
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <fstream>
#include <iostream>
#include <map>
#include <sstream>
#include <string>
#include <type_traits>
#include <vector>

#include <plog/Appenders/ConsoleAppender.h>
#include "path.h"
#include "logging.h"
#include "modelSpecInternal.h"
#include "code_generator/generateMakefile.h"
#include "code_generator/generateModules.h"
#include "code_generator/modelSpecMerged.h"
#include "runtime/runtime.h"
#include "optimiser.h"

using namespace GeNN;
// The same driver runs the network on the MI355X backend when built with -DDRIVER_BACKEND_MI355X (and the
// include path of that backend's optimiser.h first); array layouts are converted to the backend's row stride.
#ifdef DRIVER_BACKEND_MI355X
using namespace GeNN::CodeGenerator::MI355X;
#else
using namespace GeNN::CodeGenerator::SingleThreadedCPU;
#endif

// ---------------------------------------------------------------------------------------------
// Models that are not built into the reference (declared the way a user of its C++ API would)
// ---------------------------------------------------------------------------------------------
// All-to-all trace STDP: the "stdp_additive_2" example of pygenn/genn_model.py:1448-1476
class TraceSTDP : public WeightUpdateModels::Base
{
public:
    DECLARE_SNIPPET(TraceSTDP);
    SET_PARAMS({"tauPlus", "tauMinus", "aPlus", "aMinus", "wMin", "wMax"});
    SET_DERIVED_PARAMS({
        {"tauPlusDecay", [](const ParamValues &p, double dt){ return std::exp(-dt / p.at("tauPlus").cast<double>()); }},
        {"tauMinusDecay", [](const ParamValues &p, double dt){ return std::exp(-dt / p.at("tauMinus").cast<double>()); }}});
    SET_VARS({{"g", "scalar"}});
    SET_PRE_VARS({{"preTrace", "scalar"}});
    SET_POST_VARS({{"postTrace", "scalar"}});
    SET_PRE_SPIKE_SYN_CODE(
        "addToPost(g);\n"
        "const scalar dt = t - st_post;\n"
        "if(dt > 0) {\n"
        "    const scalar newWeight = g - (aMinus * postTrace);\n"
        "    g = fmin(wMax, fmax(wMin, newWeight));\n"
        "}\n");
    SET_POST_SPIKE_SYN_CODE(
        "const scalar dt = t - st_pre;\n"
        "if(dt > 0) {\n"
        "    const scalar newWeight = g + (aPlus * preTrace);\n"
        "    g = fmin(wMax, fmax(wMin, newWeight));\n"
        "}\n");
    SET_PRE_SPIKE_CODE("preTrace += 1.0;\n");
    SET_PRE_DYNAMICS_CODE("preTrace *= tauPlusDecay;\n");
    SET_POST_SPIKE_CODE("postTrace += 1.0;\n");
    SET_POST_DYNAMICS_CODE("postTrace *= tauMinusDecay;\n");
};
IMPLEMENT_SNIPPET(TraceSTDP);

// The built-in WeightUpdateModels::StaticGraded (weightUpdateModels.h:308-319) with one identifier changed: its event code
// reads the presynaptic potential as `V_pre`, but the 5.4.0 code generator exposes a presynaptic neuron variable reference
// under its own name (`V`; synapseUpdateGroupMerged.cc:62-69), so the built-in does not transpile ("Undefined identifier"
// at 'V_pre').  Everything else is the built-in's.
class GradedSynapse : public WeightUpdateModels::Base
{
public:
    DECLARE_SNIPPET(GradedSynapse);
    SET_PARAMS({"Epre", "Vslope"});
    SET_VARS({{"g", "scalar", VarAccess::READ_ONLY}});
    SET_PRE_NEURON_VAR_REFS({{"V", "scalar", VarAccessMode::READ_ONLY}});
    SET_PRE_EVENT_THRESHOLD_CONDITION_CODE("V > Epre");
    SET_PRE_EVENT_SYN_CODE("addToPost(fmax(0.0, g * tanh((V - Epre) / Vslope) * dt));\n");
};
IMPLEMENT_SNIPPET(GradedSynapse);

// Presynaptic ("reverse") output: the static_pulse_reverse model of tests/features/test_event_propagation.py:584-590
class StaticPulseReverse : public WeightUpdateModels::Base
{
public:
    DECLARE_SNIPPET(StaticPulseReverse);
    SET_VARS({{"g", "scalar", VarAccess::READ_ONLY}});
    SET_PRE_SPIKE_SYN_CODE("addToPre(g);\n");
};
IMPLEMENT_SNIPPET(StaticPulseReverse);

// Models no backend has built in (what a user of the API writes): they reach the MI355X backend's generated kernels.
// LIF with a spike-triggered adaptation current: the built-in LIF (neuronModels.h:220-257) plus one state variable that
// decays every step, is subtracted from the input and grows at every spike.
class LIFAdapt : public NeuronModels::Base
{
public:
    DECLARE_SNIPPET(LIFAdapt);
    SET_SIM_CODE(
        "if (RefracTime <= 0.0) {\n"
        "  scalar alpha = ((Isyn + Ioffset - A) * Rmembrane) + Vrest;\n"
        "  V = alpha - (ExpTC * (alpha - V));\n"
        "}\n"
        "else {\n"
        "  RefracTime -= dt;\n"
        "}\n"
        "A *= ExpA;\n");
    SET_THRESHOLD_CONDITION_CODE("RefracTime <= 0.0 && V >= Vthresh");
    SET_RESET_CODE(
        "V = Vreset;\n"
        "RefracTime = TauRefrac;\n"
        "A += dA;\n");
    SET_PARAMS({"C", "TauM", "Vrest", "Vreset", "Vthresh", "Ioffset", "TauRefrac", "TauA", "dA"});
    SET_DERIVED_PARAMS({
        {"ExpTC", [](const ParamValues &pars, double dt){ return std::exp(-dt / pars.at("TauM").cast<double>()); }},
        {"Rmembrane", [](const ParamValues &pars, double){ return pars.at("TauM").cast<double>() / pars.at("C").cast<double>(); }},
        {"ExpA", [](const ParamValues &pars, double dt){ return std::exp(-dt / pars.at("TauA").cast<double>()); }}});
    SET_VARS({{"V", "scalar"}, {"RefracTime", "scalar"}, {"A", "scalar"}});
    SET_NEEDS_AUTO_REFRACTORY(false);
};
IMPLEMENT_SNIPPET(LIFAdapt);

// Weight update model with presynaptic and postsynaptic variables, after the models of tests/features/test_wu_vars.py:
// each neuron's variable takes the time of its last spike (pre / post spike code, run in the neuron update); a
// presynaptic spike delivers g and copies the target's variable into its synapses, a postsynaptic spike copies the
// source's variable into its column (learnPost).
class TimingCopy : public WeightUpdateModels::Base
{
public:
    DECLARE_SNIPPET(TimingCopy);
    SET_VARS({{"g", "scalar", VarAccess::READ_ONLY}, {"wPre", "scalar"}, {"wPost", "scalar"}});
    SET_PRE_VARS({{"sPre", "scalar"}});
    SET_POST_VARS({{"sPost", "scalar"}});
    SET_PRE_SPIKE_CODE("sPre = t;\n");
    SET_POST_SPIKE_CODE("sPost = t;\n");
    SET_PRE_SPIKE_SYN_CODE(
        "addToPost(g);\n"
        "wPost = sPost;\n");
    SET_POST_SPIKE_SYN_CODE("wPre = sPre;\n");
};
IMPLEMENT_SNIPPET(TimingCopy);

// The same idea with the times GeNN keeps itself: a presynaptic spike delivers g and writes the time of the target's spike
// BEFORE its latest one into the row's synapses, a postsynaptic spike writes the source's into its column (prev_st_post /
// prev_st_pre: both populations then keep previous spike times, updated by a kernel of their own on the SIMT backends).
class PrevTiming : public WeightUpdateModels::Base
{
public:
    DECLARE_SNIPPET(PrevTiming);
    SET_VARS({{"g", "scalar", VarAccess::READ_ONLY}, {"wPre", "scalar"}, {"wPost", "scalar"}});
    SET_PRE_SPIKE_SYN_CODE(
        "addToPost(g);\n"
        "wPost = prev_st_post;\n");
    SET_POST_SPIKE_SYN_CODE("wPre = prev_st_pre;\n");
};
IMPLEMENT_SNIPPET(PrevTiming);

// Weight update model that runs EVERY step for EVERY synapse (synapse dynamics code), after the continuous models of
// tests/features/test_synapse_dynamics*.py: each synapse low-pass filters how far its source's membrane potential is above a
// midpoint and delivers g times that trace, spike or no spike.
class LeakyGraded : public WeightUpdateModels::Base
{
public:
    DECLARE_SNIPPET(LeakyGraded);
    SET_PARAMS({"Vmid", "decay"});
    SET_VARS({{"g", "scalar", VarAccess::READ_ONLY}, {"x", "scalar"}});
    SET_PRE_NEURON_VAR_REFS({{"Vpre", "scalar", VarAccessMode::READ_ONLY}});
    SET_SYNAPSE_DYNAMICS_CODE(
        "x = (x * decay) + fmax(0.0, Vpre - Vmid);\n"
        "addToPost(g * x);\n");
};
IMPLEMENT_SNIPPET(LeakyGraded);

// Postsynaptic spike-like events (after tests/features/test_event_propagation.py): while a target's membrane potential is above
// a midpoint, every synapse onto it counts the step in a variable of its own and sends a fraction of its weight back to its
// source (addToPre), next to ordinary forward transmission.
class PostEventFeedback : public WeightUpdateModels::Base
{
public:
    DECLARE_SNIPPET(PostEventFeedback);
    SET_PARAMS({"Vmid", "back"});
    SET_VARS({{"g", "scalar", VarAccess::READ_ONLY}, {"hits", "scalar"}});
    SET_POST_NEURON_VAR_REFS({{"Vpost", "scalar", VarAccessMode::READ_ONLY}});
    SET_PRE_SPIKE_SYN_CODE("addToPost(g);\n");
    SET_POST_EVENT_THRESHOLD_CONDITION_CODE("Vpost > Vmid");
    SET_POST_EVENT_SYN_CODE(
        "hits += 1.0;\n"
        "addToPre(back * g);\n");
};
IMPLEMENT_SNIPPET(PostEventFeedback);

// Synapses that release with a probability: random numbers in weight-update code (what a user writes for stochastic
// transmission; cf. tests/features/test_rng.py, which draws in neuron code).
class StochasticPulse : public WeightUpdateModels::Base
{
public:
    DECLARE_SNIPPET(StochasticPulse);
    SET_PARAMS({"pRelease"});
    SET_VARS({{"g", "scalar", VarAccess::READ_ONLY}});
    SET_PRE_SPIKE_SYN_CODE(
        "if(gennrand_uniform() < pRelease) {\n"
        "    addToPost(g);\n"
        "}\n");
};
IMPLEMENT_SNIPPET(StochasticPulse);

// Current source fed from a host-pregenerated array; the driver rewrites the N-element
// window before every step, so the injected value at step s is noise[s*N + id].
class ArrayNoise : public CurrentSourceModels::Base
{
public:
    DECLARE_SNIPPET(ArrayNoise);
    SET_INJECTION_CODE("injectCurrent(noise[id]);\n");
    SET_EXTRA_GLOBAL_PARAMS({{"noise", "scalar*"}});
};
IMPLEMENT_SNIPPET(ArrayNoise);

// Custom updates (functions a user calls between steps, Runtime::customUpdate), after tests/features/test_custom_update.py:
// a per-neuron one that pulls a referenced variable towards a rest value and counts its calls in a variable of its own;
class DecayToRest : public CustomUpdateModels::Base
{
public:
    DECLARE_SNIPPET(DecayToRest);
    SET_PARAMS({"rest", "factor"});
    SET_CUSTOM_UPDATE_VARS({{"applied", "scalar", CustomUpdateVarAccess::READ_WRITE}});
    SET_VAR_REFS({{"v", "scalar", VarAccessMode::READ_WRITE}});
    SET_UPDATE_CODE(
        "v = rest + ((v - rest) * factor);\n"
        "applied += 1.0;\n");
};
IMPLEMENT_SNIPPET(DecayToRest);

// a reduction over the neurons of a population: sum and maximum of a referenced variable, one value each per batch;
class NeuronSumMax : public CustomUpdateModels::Base
{
public:
    DECLARE_SNIPPET(NeuronSumMax);
    SET_CUSTOM_UPDATE_VARS({{"sum", "scalar", CustomUpdateVarAccess::REDUCE_NEURON_SUM}, {"peak", "scalar", CustomUpdateVarAccess::REDUCE_NEURON_MAX}});
    SET_VAR_REFS({{"v", "scalar", VarAccessMode::READ_ONLY}});
    SET_UPDATE_CODE(
        "sum = v;\n"
        "peak = v;\n");
};
IMPLEMENT_SNIPPET(NeuronSumMax);

// a per-synapse one: weight decay with the decayed weight accumulated in a variable of its own, every `t`-dependence
// included so that the time the function is handed shows (the time of the step the model has reached);
class WeightDecay : public CustomUpdateModels::Base
{
public:
    DECLARE_SNIPPET(WeightDecay);
    SET_PARAMS({"factor"});
    SET_CUSTOM_UPDATE_VARS({{"total", "scalar", CustomUpdateVarAccess::READ_WRITE}, {"when", "scalar", CustomUpdateVarAccess::READ_WRITE}});
    SET_VAR_REFS({{"w", "scalar", VarAccessMode::READ_WRITE}});
    SET_UPDATE_CODE(
        "w *= factor;\n"
        "total += w;\n"
        "when = t + (0.001 * id_pre) + (1000.0 * id_post);\n");
};
IMPLEMENT_SNIPPET(WeightDecay);

// a reduction over batches: the sum and the maximum of a per-batch synaptic variable (what gradient accumulation does)
class BatchSumMax : public CustomUpdateModels::Base
{
public:
    DECLARE_SNIPPET(BatchSumMax);
    SET_CUSTOM_UPDATE_VARS({{"sum", "scalar", CustomUpdateVarAccess::REDUCE_BATCH_SUM}, {"peak", "scalar", CustomUpdateVarAccess::REDUCE_BATCH_MAX}});
    SET_VAR_REFS({{"w", "scalar", VarAccessMode::READ_ONLY}});
    SET_UPDATE_CODE(
        "sum = w;\n"
        "peak = w;\n");
};
IMPLEMENT_SNIPPET(BatchSumMax);

// Custom connectivity updates (structural plasticity: a function of the model that rewires a SPARSE projection between steps),
// after tests/features/test_custom_connectivity_update.py: one that removes every synapse whose weight has fallen below a
// threshold (set per row by host update code) and counts the removals of its row in a presynaptic variable of its own;
class PruneWeak : public CustomConnectivityUpdateModels::Base
{
public:
    DECLARE_SNIPPET(PruneWeak);
    SET_PARAMS({"threshold"});
    SET_PRE_VARS({{"removed", "scalar"}, {"limit", "scalar"}});
    SET_VAR_REFS({{"w", "scalar", VarAccessMode::READ_ONLY}});
    // (the threshold of a row is set by host code that runs before the rows are walked, and rises with the row and the time)
    SET_HOST_UPDATE_CODE(
        "for(unsigned int i = 0; i < num_pre; i++) {\n"
        "    limit[i] = threshold + (0.0001 * i) + (0.00005 * t);\n"
        "}\n"
        "pushlimitToDevice();\n");
    SET_ROW_UPDATE_CODE(
        "for_each_synapse {\n"
        "    if(w < limit) {\n"
        "        remove_synapse();\n"
        "        removed += 1.0;\n"
        "    }\n"
        "}\n");
};
IMPLEMENT_SNIPPET(PruneWeak);

// and one that gives every row that has room a new synapse onto a target that moves on with every call (rows start apart, so
// that columns fill evenly), with a weight the
// call fixes and a per-synapse variable of its own that records when the synapse was made (older synapses keep theirs)
class Sprout : public CustomConnectivityUpdateModels::Base
{
public:
    DECLARE_SNIPPET(Sprout);
    SET_PARAMS({"weight"});
    SET_VARS({{"born", "scalar"}});
    SET_PRE_VARS({{"next", "unsigned int"}});
    SET_VAR_REFS({{"w", "scalar", VarAccessMode::READ_WRITE}});
    SET_ROW_UPDATE_CODE(
        "const unsigned int target = (next + (3 * id_pre)) % num_post;\n"
        "bool present = false;\n"
        "for_each_synapse {\n"
        "    if(id_post == target) {\n"
        "        present = true;\n"
        "        break;\n"
        "    }\n"
        "}\n"
        "if(!present && row_length < row_stride) {\n"
        "    add_synapse(target, t, weight);\n"
        "}\n"
        "next = (next + 7) % num_post;\n");
};
IMPLEMENT_SNIPPET(Sprout);

// ---------------------------------------------------------------------------------------------
template<typename T>
static std::vector<T> readFile(const std::string &path, size_t expect = 0)
{
    std::ifstream f(path, std::ios::binary | std::ios::ate);
    if(!f) { throw std::runtime_error("cannot open " + path); }
    const size_t bytes = (size_t)f.tellg();
    f.seekg(0);
    std::vector<T> v(bytes / sizeof(T));
    f.read(reinterpret_cast<char*>(v.data()), bytes);
    if(expect && v.size() != expect) {
        throw std::runtime_error(path + ": expected " + std::to_string(expect) + " elements, got " + std::to_string(v.size()));
    }
    return v;
}

template<typename T>
static void appendFile(const std::string &path, const T *data, size_t n)
{
    std::ofstream f(path, std::ios::binary | std::ios::app);
    f.write(reinterpret_cast<const char*>(data), n * sizeof(T));
}

struct PopSpec { std::string name, model; unsigned int n; std::vector<double> p; NeuronGroup *ng = nullptr; };
struct CSSpec { std::string name, model, pop; std::vector<double> p; CurrentSource *cs = nullptr; };
struct DynamicSpec { std::string kind, group, param; unsigned int step; double value; };     // a parameter set while the model runs
struct SynSpec
{
    std::string name, matrix, src, trg, wum, psm, connect, initSnippet;
    double connectValue = 0.0;
    unsigned int rowStride = 0, maxDenDelay = 0, tps = 1, colStride = 0, axonalDelay = 0;
    bool hintPre = false;
    std::vector<double> conv, wumP, psmP;
    SynapseGroup *sg = nullptr;
};

// Arrays of the model's scalar type hold float or double (--precision=double); the netspec's files and the dumps are fp32 either way
static void appendScalars(const std::string &path, Runtime::ArrayBase *a, size_t first, size_t count)
{
    if(a->getType() == Type::Double) {
        const double *src = a->getHostPointer<double>() + first;
        std::vector<float> narrow(src, src + count);
        appendFile(path, narrow.data(), count);
    }
    else {
        appendFile(path, a->getHostPointer<float>() + first, count);
    }
}
static void storeScalars(Runtime::ArrayBase *a, size_t first, const float *src, size_t count)
{
    if(a->getType() == Type::Double) { std::copy_n(src, count, a->getHostPointer<double>() + first); }
    else { std::copy_n(src, count, a->getHostPointer<float>() + first); }
}

// custom <name> <update group> <kind> <target> [<second target>] [<params>]; custom_call <update group> <every n steps>
struct CustomSpec
{
    std::string name, group, kind, target, target2;
    std::vector<double> p;
    CustomUpdate *cu = nullptr;
    CustomUpdateWU *cuWU = nullptr;
    CustomConnectivityUpdate *ccu = nullptr;
};
struct CustomCallSpec { std::string group; unsigned int every; };

int main(int argc, char *argv[])
{
    try {
        if(argc < 4) { std::cerr << "usage: ref_driver <netspec dir> <work dir> <out dir> [--generate-only] [--cxxflags=<flags>]" << std::endl; return 1; }
        const std::string in = argv[1], work = argv[2], out = argv[3];
        bool generateOnly = false;
        std::string userCxxFlags;
        std::vector<std::string> dynamicParams;
        bool timing = false, ordered = false, deviceInit = false, doublePrecision = false, narrowInd = false, deviceArrays = false, profilerRanges = false, zeroCopyRecording = false;
        int stepQueue = -1;
        std::string kernels = "auto";
        for(int a = 4; a < argc; a++) {
            const std::string opt = argv[a];
            if(opt == "--generate-only") { generateOnly = true; }
            else if(opt.rfind("--cxxflags=", 0) == 0) { userCxxFlags = opt.substr(11); }      // e.g. -O3: same results as the default build, faster
            // --dynamic=neuron:<population>.<param> | cs:<source>.<param> | wu:<projection>.<param> | ps:<projection>.<param>: marks a
            // parameter dynamic (setParamDynamic and friends), as a model that calls setDynamicParamValue at run time would
            else if(opt.rfind("--dynamic=", 0) == 0) { dynamicParams.push_back(opt.substr(10)); }
            else if(opt.rfind("--kernels=", 0) == 0) { kernels = opt.substr(10); }    // MI355X backend: library | generated | auto (Preferences::kernelSource)
            else if(opt.rfind("--step-queue=", 0) == 0) { stepQueue = std::stoi(opt.substr(13)); }      // MI355X backend: Preferences::stepQueueLength
            else if(opt == "--zero-copy-recording") { zeroCopyRecording = true; }  // NeuronGroup::setRecordingZeroCopyEnabled for every population
            else if(opt == "--profiler-ranges") { profilerRanges = true; }         // MI355X backend: Preferences::profilerRanges
            else if(opt == "--device-init") { deviceInit = true; }                  // MI355X backend: Preferences::deviceInitialisation
            // matrices built by snippets are placed on the device only (VarLocation::DEVICE) and not written to the out directory
            else if(opt == "--device-arrays") { deviceArrays = true; }
            else if(opt == "--ordered") { ordered = true; }                          // MI355X backend: Preferences::orderedAccumulation
            else if(opt == "--narrow-ind") { narrowInd = true; }     // ModelSpec::setDefaultNarrowSparseIndEnabled; for --generate-only runs (the netspec's targets are 32-bit)
            else if(opt == "--precision=double") { doublePrecision = true; }        // ModelSpec::setPrecision(Type::Double); for --generate-only runs (the netspec's arrays are fp32)
            else if(opt == "--timing") { timing = true; }       // ModelSpec::setTimingEnabled; the Runtime's counters are printed after the run
            else { std::cerr << "unknown option " << opt << std::endl; return 1; }
        }

        plog::ConsoleAppender<plog::TxtFormatter> app;
        Preferences prefs;
        prefs.userCxxFlagsGNU = userCxxFlags;
#ifdef DRIVER_BACKEND_MI355X
        prefs.kernelSource = (kernels == "generated") ? Preferences::KernelSource::GENERATED : (kernels == "library") ? Preferences::KernelSource::LIBRARY : Preferences::KernelSource::AUTO;
        prefs.orderedAccumulation = ordered;
        if(stepQueue >= 0) { prefs.stepQueueLength = (unsigned int)stepQueue; }
        prefs.deviceInitialisation = deviceInit;
        prefs.profilerRanges = profilerRanges;
#else
        (void)ordered; (void)stepQueue; (void)deviceInit; (void)profilerRanges;
#endif
        Logging::init(prefs.gennLogLevel, prefs.codeGeneratorLogLevel, prefs.transpilerLogLevel,
                      prefs.runtimeLogLevel, &app, &app, &app, &app);

        // ---- parse net.txt -----------------------------------------------------------------
        std::string name = "net";
        double dt = 1.0;
        unsigned int steps = 1, snap = 0, fuse = 0, batch = 1, seed = 0;
        std::vector<PopSpec> pops; std::vector<CSSpec> css; std::vector<SynSpec> syns; std::vector<DynamicSpec> dynamics;
        std::vector<CustomSpec> customs; std::vector<CustomCallSpec> customCalls;
        {
            std::ifstream f(in + "/net.txt");
            if(!f) { throw std::runtime_error("no net.txt in " + in); }
            std::string line;
            while(std::getline(f, line)) {
                std::istringstream ls(line);
                std::string k; if(!(ls >> k) || k[0] == '#') { continue; }
                if(k == "model") ls >> name;
                else if(k == "dt") ls >> dt;
                else if(k == "steps") ls >> steps;
                else if(k == "snap") ls >> snap;
                else if(k == "fuse_psm") ls >> fuse;
                else if(k == "batch") ls >> batch;
                else if(k == "seed") ls >> seed;
                else if(k == "precision") { std::string v; ls >> v; doublePrecision = (v == "double"); }      // ModelSpec::setPrecision
                else if(k == "dynamic") { DynamicSpec d; ls >> d.kind >> d.group >> d.param >> d.step >> d.value; dynamics.push_back(d); dynamicParams.push_back(d.kind + ":" + d.group + "." + d.param); }
                else if(k == "pop") { PopSpec p; ls >> p.name >> p.model >> p.n; double v; while(ls >> v) p.p.push_back(v); pops.push_back(p); }
                else if(k == "cs") { CSSpec c; ls >> c.name >> c.model >> c.pop; double v; while(ls >> v) c.p.push_back(v); css.push_back(c); }
                else if(k == "syn") {
                    SynSpec s; ls >> s.name >> s.matrix >> s.src >> s.trg;
                    if(s.matrix == "sparse") { ls >> s.rowStride; }
                    else if(s.matrix == "conv2d") { s.conv.resize(8); for(auto &c : s.conv) ls >> c; }
                    // Conv2D as SPARSE connectivity: kh kw sh sw padh padw ih iw ic oh ow oc (initSparseConnectivitySnippet.h:438-497)
                    else if(s.matrix == "conv2d_sparse") { s.conv.resize(12); for(auto &c : s.conv) ls >> c; }
                    else if(s.matrix == "procedural" || s.matrix == "sparse_init") { ls >> s.connect >> s.connectValue; }
                    // ("dense_init": a stored DENSE matrix whose weights an initialisation snippet draws, wum static_init)
                    else if(s.matrix != "dense" && s.matrix != "dense_init" && s.matrix != "bitmask") throw std::runtime_error("matrix " + s.matrix);
                    ls >> s.wum;
                    if(s.wum == "static_init") { ls >> s.initSnippet; const int np = (s.initSnippet == "Constant") ? 1 : 2; s.wumP.resize(np); for(auto &c : s.wumP) ls >> c; }
                    if(s.wum == "static_delay") { ls >> s.maxDenDelay; }
                    else if(s.wum == "stdp_trace" || s.wum == "stdp") { s.wumP.resize(6); for(auto &c : s.wumP) ls >> c; }
                    else if(s.wum == "static_const" || s.wum == "stochastic") { s.wumP.resize(1); ls >> s.wumP[0]; }
                    else if(s.wum == "static_graded" || s.wum == "leaky_graded" || s.wum == "post_event") { s.wumP.resize(2); ls >> s.wumP[0] >> s.wumP[1]; }
                    else if(s.wum != "static" && s.wum != "static_reverse" && s.wum != "static_init" && s.wum != "static_kernel" && s.wum != "timing_copy" && s.wum != "prev_timing") throw std::runtime_error("wum " + s.wum);
                    ls >> s.psm;
                    if(s.psm == "expcurr") { s.psmP.resize(1); ls >> s.psmP[0]; }
                    else if(s.psm != "deltacurr") throw std::runtime_error("psm " + s.psm);
                    std::string o;
                    while(ls >> o) { if(o == "hint_pre") s.hintPre = true; else if(o == "tps") ls >> s.tps; else if(o == "col_stride") ls >> s.colStride; else if(o == "axonal_delay") ls >> s.axonalDelay; else throw std::runtime_error("opt " + o); }
                    syns.push_back(s);
                }
                else if(k == "custom") {
                    CustomSpec c; ls >> c.name >> c.group >> c.kind >> c.target;
                    if(c.kind == "transpose") { ls >> c.target2; }
                    double v; while(ls >> v) c.p.push_back(v);
                    customs.push_back(c);
                }
                else if(k == "custom_call") { CustomCallSpec c; ls >> c.group >> c.every; customCalls.push_back(c); }
                else throw std::runtime_error("unknown key " + k);
            }
        }

        // ---- build ModelSpec ---------------------------------------------------------------
        ModelSpecInternal model;
        model.setName(name);
        model.setDT(dt);
        model.setBatchSize(batch);
        if(seed) { model.setSeed(seed); }
        model.setPrecision(doublePrecision ? Type::Double : Type::Float);
        model.setFusePostsynapticModels(fuse != 0);
        model.setDefaultNarrowSparseIndEnabled(narrowInd);
        model.setTimingEnabled(timing);
        std::map<std::string, PopSpec*> popByName;
        for(auto &p : pops) {
            if(p.model == "lif") {
                p.ng = model.addNeuronPopulation<NeuronModels::LIF>(p.name, p.n,
                    {{"C", p.p.at(0)}, {"TauM", p.p.at(1)}, {"Vrest", p.p.at(2)}, {"Vreset", p.p.at(3)},
                     {"Vthresh", p.p.at(4)}, {"Ioffset", p.p.at(5)}, {"TauRefrac", p.p.at(6)}},
                    {{"V", uninitialisedVar()}, {"RefracTime", uninitialisedVar()}});
            }
            else if(p.model == "lif_init") {
                // the membrane potential by an initialisation snippet instead of a file
                p.ng = model.addNeuronPopulation<NeuronModels::LIF>(p.name, p.n,
                    {{"C", p.p.at(0)}, {"TauM", p.p.at(1)}, {"Vrest", p.p.at(2)}, {"Vreset", p.p.at(3)},
                     {"Vthresh", p.p.at(4)}, {"Ioffset", p.p.at(5)}, {"TauRefrac", p.p.at(6)}},
                    {{"V", initVar<InitVarSnippet::Uniform>({{"min", p.p.at(7)}, {"max", p.p.at(8)}})}, {"RefracTime", 0.0}});
            }
            else if(p.model == "lifa") {
                p.ng = model.addNeuronPopulation<LIFAdapt>(p.name, p.n,
                    {{"C", p.p.at(0)}, {"TauM", p.p.at(1)}, {"Vrest", p.p.at(2)}, {"Vreset", p.p.at(3)},
                     {"Vthresh", p.p.at(4)}, {"Ioffset", p.p.at(5)}, {"TauRefrac", p.p.at(6)}, {"TauA", p.p.at(7)}, {"dA", p.p.at(8)}},
                    {{"V", uninitialisedVar()}, {"RefracTime", uninitialisedVar()}, {"A", uninitialisedVar()}});
            }
            else if(p.model == "izh") {
                p.ng = model.addNeuronPopulation<NeuronModels::Izhikevich>(p.name, p.n,
                    {{"a", p.p.at(0)}, {"b", p.p.at(1)}, {"c", p.p.at(2)}, {"d", p.p.at(3)}},
                    {{"V", uninitialisedVar()}, {"U", uninitialisedVar()}});
            }
            else if(p.model == "poisson") {
                p.ng = model.addNeuronPopulation<NeuronModels::Poisson>(p.name, p.n, {{"rate", p.p.at(0)}}, {{"timeStepToSpike", uninitialisedVar()}});
            }
            else if(p.model == "ssa") {
                p.ng = model.addNeuronPopulation<NeuronModels::SpikeSourceArray>(p.name, p.n, {},
                    {{"startSpike", uninitialisedVar()}, {"endSpike", uninitialisedVar()}});
            }
            else throw std::runtime_error("pop model " + p.model);
            p.ng->setSpikeRecordingEnabled(true);
            if(zeroCopyRecording) { p.ng->setRecordingZeroCopyEnabled(true); }
            popByName[p.name] = &p;
        }
        // populations that drive graded projections also record their spike-like events
        for(auto &s : syns) { if(s.wum == "static_graded") { popByName.at(s.src)->ng->setSpikeEventRecordingEnabled(true); } }
        for(auto &c : css) {
            NeuronGroup *ng = popByName.at(c.pop)->ng;
            if(c.model == "dc") c.cs = model.addCurrentSource<CurrentSourceModels::DC>(c.name, ng, {{"amp", c.p.at(0)}}, {});
            else if(c.model == "noise") c.cs = model.addCurrentSource<ArrayNoise>(c.name, ng, {}, {});
            else if(c.model == "poisson_exp") {
                c.cs = model.addCurrentSource<CurrentSourceModels::PoissonExp>(c.name, ng, {{"weight", c.p.at(0)}, {"tauSyn", c.p.at(1)}, {"rate", c.p.at(2)}}, {{"current", 0.0}});
            }
            else throw std::runtime_error("cs model " + c.model);
        }
        for(auto &s : syns) {
            NeuronGroup *src = popByName.at(s.src)->ng, *trg = popByName.at(s.trg)->ng;
            const auto psm = (s.psm == "expcurr") ? initPostsynaptic<PostsynapticModels::ExpCurr>({{"tau", s.psmP[0]}})
                                                  : initPostsynaptic<PostsynapticModels::DeltaCurr>();
            WeightUpdateModels::Init wum = initWeightUpdate<WeightUpdateModels::StaticPulse>({}, {{"g", uninitialisedVar()}});
            if(s.wum == "static_const") {
                wum = initWeightUpdate<WeightUpdateModels::StaticPulseConstantWeight>({{"g", s.wumP[0]}});
            }
            else if(s.wum == "static_reverse") {
                wum = initWeightUpdate<StaticPulseReverse>({}, {{"g", uninitialisedVar()}});
            }
            else if(s.wum == "stochastic") {
                wum = initWeightUpdate<StochasticPulse>({{"pRelease", s.wumP.at(0)}}, {{"g", uninitialisedVar()}});
            }
            else if(s.wum == "leaky_graded") {
                wum = initWeightUpdate<LeakyGraded>({{"Vmid", s.wumP.at(0)}, {"decay", s.wumP.at(1)}}, {{"g", uninitialisedVar()}, {"x", 0.0}}, {}, {},
                                                    {{"Vpre", createVarRef(popByName.at(s.src)->ng, "V")}}, {});
            }
            else if(s.wum == "post_event") {
                wum = initWeightUpdate<PostEventFeedback>({{"Vmid", s.wumP.at(0)}, {"back", s.wumP.at(1)}}, {{"g", uninitialisedVar()}, {"hits", 0.0}}, {}, {},
                                                          {}, {{"Vpost", createVarRef(popByName.at(s.trg)->ng, "V")}});
            }
            else if(s.wum == "prev_timing") {
                wum = initWeightUpdate<PrevTiming>({}, {{"g", uninitialisedVar()}, {"wPre", -1.0}, {"wPost", -1.0}});
            }
            else if(s.wum == "timing_copy") {
                wum = initWeightUpdate<TimingCopy>({}, {{"g", uninitialisedVar()}, {"wPre", 0.0}, {"wPost", 0.0}}, {{"sPre", 0.0}}, {{"sPost", 0.0}});
            }
            else if(s.wum == "static_graded") {
                const ParamValues gradedParams{{"Epre", s.wumP[0]}, {"Vslope", s.wumP[1]}};
                const VarValues gradedVars{{"g", uninitialisedVar()}};
#ifdef DRIVER_BACKEND_MI355X
                // the adapter recognises the built-in as it stands (its library path never transpiles the event code); kernels
                // generated from the code need the variant that transpiles
                if(kernels != "generated") { wum = initWeightUpdate<WeightUpdateModels::StaticGraded>(gradedParams, gradedVars, {}, {}, {{"V", std::string("V")}}); }
                else
#endif
                { wum = initWeightUpdate<GradedSynapse>(gradedParams, gradedVars, {}, {}, {{"V", std::string("V")}}); }
            }
            else if(s.wum == "static_delay") {
                wum = initWeightUpdate<WeightUpdateModels::StaticPulseDendriticDelay>({}, {{"g", uninitialisedVar()}, {"d", uninitialisedVar()}});
            }
            else if(s.wum == "stdp_trace") {
                wum = initWeightUpdate<TraceSTDP>(
                    {{"tauPlus", s.wumP[0]}, {"tauMinus", s.wumP[1]}, {"aPlus", s.wumP[2]}, {"aMinus", s.wumP[3]}, {"wMin", s.wumP[4]}, {"wMax", s.wumP[5]}},
                    {{"g", uninitialisedVar()}}, {{"preTrace", uninitialisedVar()}}, {{"postTrace", uninitialisedVar()}});
            }
            else if(s.wum == "stdp") {
                wum = initWeightUpdate<WeightUpdateModels::STDP>(
                    {{"tauPlus", s.wumP[0]}, {"tauMinus", s.wumP[1]}, {"Aplus", s.wumP[2]}, {"Aminus", s.wumP[3]}, {"Wmin", s.wumP[4]}, {"Wmax", s.wumP[5]}},
                    {{"g", uninitialisedVar()}});
            }
            if(s.wum == "static_init") {
                const auto init = (s.initSnippet == "Constant") ? initVar<InitVarSnippet::Constant>({{"constant", s.wumP[0]}})
                                : (s.initSnippet == "Uniform") ? initVar<InitVarSnippet::Uniform>({{"min", s.wumP[0]}, {"max", s.wumP[1]}})
                                : initVar<InitVarSnippet::Normal>({{"mean", s.wumP[0]}, {"sd", s.wumP[1]}});
                wum = initWeightUpdate<WeightUpdateModels::StaticPulse>({}, {{"g", init}});
            }
            if(s.wum == "static_kernel") {
                // every weight is the entry of <name>.kernel.f32 that the synapse's position in the kernel names
                wum = initWeightUpdate<WeightUpdateModels::StaticPulse>({}, {{"g", initVar<InitVarSnippet::Kernel>()}});
            }
            if(s.matrix == "conv2d_sparse") {
                s.sg = model.addSynapsePopulation(s.name, SynapseMatrixType::SPARSE, src, trg, wum, psm,
                    initConnectivity<InitSparseConnectivitySnippet::Conv2D>(
                        {{"conv_kh", (int)s.conv[0]}, {"conv_kw", (int)s.conv[1]}, {"conv_sh", (int)s.conv[2]}, {"conv_sw", (int)s.conv[3]},
                         {"conv_padh", (int)s.conv[4]}, {"conv_padw", (int)s.conv[5]}, {"conv_ih", (int)s.conv[6]}, {"conv_iw", (int)s.conv[7]},
                         {"conv_ic", (int)s.conv[8]}, {"conv_oh", (int)s.conv[9]}, {"conv_ow", (int)s.conv[10]}, {"conv_oc", (int)s.conv[11]}}));
            }
            else if(s.matrix == "procedural" || s.matrix == "sparse_init") {
                const auto connect = (s.connect == "FixedNumberPostWithReplacement")
                    ? initConnectivity<InitSparseConnectivitySnippet::FixedNumberPostWithReplacement>({{"num", (unsigned int)s.connectValue}})
                    : (s.connect == "FixedNumberPreWithReplacement")
                    ? initConnectivity<InitSparseConnectivitySnippet::FixedNumberPreWithReplacement>({{"num", (unsigned int)s.connectValue}})
                    : (s.connect == "FixedProbabilityNoAutapse") ? initConnectivity<InitSparseConnectivitySnippet::FixedProbabilityNoAutapse>({{"prob", s.connectValue}})
                    : initConnectivity<InitSparseConnectivitySnippet::FixedProbability>({{"prob", s.connectValue}});
                // ("sparse_init": the same snippets initialise a stored SPARSE matrix)
                s.sg = model.addSynapsePopulation(s.name, (s.matrix == "procedural") ? SynapseMatrixType::PROCEDURAL : SynapseMatrixType::SPARSE, src, trg, wum, psm, connect);
            }
            else if(s.matrix == "sparse") {
                s.sg = model.addSynapsePopulation(s.name, SynapseMatrixType::SPARSE, src, trg, wum, psm);
                s.sg->setMaxConnections(s.rowStride);
                if(s.colStride) s.sg->setMaxSourceConnections(s.colStride);
            }
            else if(s.matrix == "dense_init") {
                s.sg = model.addSynapsePopulation(s.name, SynapseMatrixType::DENSE, src, trg, wum, psm);
            }
            else if(s.matrix == "dense") {
                // (weights given by an initialisation snippet are regenerated at every event, never stored: DENSE_PROCEDURALG)
                s.sg = model.addSynapsePopulation(s.name, (s.wum == "static_init") ? SynapseMatrixType::DENSE_PROCEDURALG : SynapseMatrixType::DENSE, src, trg, wum, psm);
            }
            else if(s.matrix == "bitmask") {
                s.sg = model.addSynapsePopulation(s.name, SynapseMatrixType::BITMASK, src, trg, wum, psm);
            }
            else {
                s.sg = model.addSynapsePopulation(s.name, SynapseMatrixType::TOEPLITZ, src, trg, wum, psm,
                    initToeplitzConnectivity<InitToeplitzConnectivitySnippet::Conv2D>(
                        {{"conv_kh", (int)s.conv[0]}, {"conv_kw", (int)s.conv[1]}, {"conv_ih", (int)s.conv[2]}, {"conv_iw", (int)s.conv[3]},
                         {"conv_ic", (int)s.conv[4]}, {"conv_oh", (int)s.conv[5]}, {"conv_ow", (int)s.conv[6]}, {"conv_oc", (int)s.conv[7]}}));
            }
            if(deviceArrays && (s.matrix == "sparse_init" || s.matrix == "conv2d_sparse")) {
                s.sg->setSparseConnectivityLocation(VarLocation::DEVICE);
                if(s.wum != "static_const") { s.sg->setWUVarLocation("g", VarLocation::DEVICE); }
            }
            if(s.maxDenDelay) s.sg->setMaxDendriticDelayTimesteps(s.maxDenDelay);
            if(s.axonalDelay) s.sg->setAxonalDelaySteps(s.axonalDelay);
            if(s.hintPre) s.sg->setParallelismHint(SynapseGroup::ParallelismHint::PRESYNAPTIC);
            if(s.tps > 1) s.sg->setNumThreadsPerSpike(s.tps);
        }
        for(const auto &spec : dynamicParams) {
            const size_t colon = spec.find(':'), dot = spec.rfind('.');
            if(colon == std::string::npos || dot == std::string::npos || dot < colon) { throw std::runtime_error("--dynamic=" + spec); }
            const std::string kind = spec.substr(0, colon), group = spec.substr(colon + 1, dot - colon - 1), param = spec.substr(dot + 1);
            bool found = false;
            if(kind == "neuron") { for(auto &p : pops) { if(p.name == group) { p.ng->setParamDynamic(param); found = true; } } }
            else if(kind == "cs") { for(auto &c : css) { if(c.name == group) { c.cs->setParamDynamic(param); found = true; } } }
            else if(kind == "wu") { for(auto &q : syns) { if(q.name == group) { q.sg->setWUParamDynamic(param); found = true; } } }
            else if(kind == "ps") { for(auto &q : syns) { if(q.name == group) { q.sg->setPSParamDynamic(param); found = true; } } }
            if(!found) { throw std::runtime_error("--dynamic=" + spec + ": no such group"); }
        }
        std::map<std::string, SynSpec*> synByName;
        for(auto &q : syns) { synByName[q.name] = &q; }
        for(auto &c : customs) {
            if(c.kind == "decay") {
                c.cu = model.addCustomUpdate<DecayToRest>(c.name, c.group, {{"rest", c.p.at(0)}, {"factor", c.p.at(1)}}, {{"applied", 0.0}},
                                                          {{"v", createVarRef(popByName.at(c.target)->ng, "V")}});
            }
            else if(c.kind == "neuron_reduce") {
                c.cu = model.addCustomUpdate<NeuronSumMax>(c.name, c.group, {}, {{"sum", 0.0}, {"peak", 0.0}},
                                                           {{"v", createVarRef(popByName.at(c.target)->ng, "V")}});
            }
            else if(c.kind == "wu_decay") {
                c.cuWU = model.addCustomUpdate<WeightDecay>(c.name, c.group, {{"factor", c.p.at(0)}}, {{"total", 0.0}, {"when", -1.0}},
                                                            WUVarReferences{{"w", createWUVarRef(synByName.at(c.target)->sg, "g")}});
            }
            else if(c.kind == "batch_reduce") {
                c.cuWU = model.addCustomUpdate<BatchSumMax>(c.name, c.group, {}, {{"sum", 0.0}, {"peak", 0.0}},
                                                            WUVarReferences{{"w", createWUVarRef(synByName.at(c.target)->sg, "g")}});
            }
            else if(c.kind == "transpose") {
                c.cuWU = model.addCustomUpdate<CustomUpdateModels::Transpose>(c.name, c.group, {}, {},
                    WUVarReferences{{"variable", createWUVarRef(synByName.at(c.target)->sg, "g", synByName.at(c.target2)->sg, "g")}});
            }
            else if(c.kind == "prune") {
                c.ccu = model.addCustomConnectivityUpdate<PruneWeak>(c.name, c.group, synByName.at(c.target)->sg, {{"threshold", c.p.at(0)}}, {}, {{"removed", 0.0}, {"limit", 0.0}}, {},
                                                                    WUVarReferences{{"w", createWUVarRef(synByName.at(c.target)->sg, "g")}}, {}, {});
            }
            else if(c.kind == "sprout") {
                c.ccu = model.addCustomConnectivityUpdate<Sprout>(c.name, c.group, synByName.at(c.target)->sg, {{"weight", c.p.at(0)}}, {{"born", -1.0}}, {{"next", 0.0}}, {},
                                                                 WUVarReferences{{"w", createWUVarRef(synByName.at(c.target)->sg, "g")}}, {}, {});
            }
            else throw std::runtime_error("custom update kind " + c.kind);
        }
        model.finalise();

        // ---- generate + build --------------------------------------------------------------
        const filesystem::path targetPath(work);
        const filesystem::path outputPath = targetPath / (model.getName() + "_CODE");
        filesystem::create_directory(outputPath);
        auto backend = Optimiser::createBackend(model, outputPath, prefs.backendLogLevel, &app, prefs);
        CodeGenerator::ModelSpecMerged modelMerged(backend, model);
        const auto moduleNames = CodeGenerator::generateAll(modelMerged, backend, outputPath, true);
        {
            std::ofstream makefile((outputPath / "Makefile").str());
            CodeGenerator::generateMakefile(makefile, backend, moduleNames);
        }
        const std::string cmd = "make -s -C \"" + outputPath.str() + "\" -j 8";
        if(system(cmd.c_str()) != 0) { throw std::runtime_error("build failed: " + cmd); }
        if(generateOnly) {
            std::cout << "ref_driver: generated and built " << outputPath.str() << std::endl;
            return 0;
        }

        // ---- run ---------------------------------------------------------------------------
        const auto startOfRun = std::chrono::steady_clock::now();
        auto sinceStart = [&startOfRun]() { return std::chrono::duration<double>(std::chrono::steady_clock::now() - startOfRun).count(); };
        Runtime::Runtime rt(targetPath, modelMerged, backend);
        rt.allocate(steps);
        const double allocated = sinceStart();
        // kernels that weights are initialised from are extra global parameters of the variable's initialiser: present before initialize()
        for(auto &s : syns) {
            if(s.wum != "static_kernel") { continue; }
            const auto kernel = readFile<float>(in + "/" + s.name + ".kernel.f32");
            rt.allocateArray(*s.sg, "kernelg", kernel.size());
            auto *a = rt.getArray(*s.sg, "kernelg");
            storeScalars(a, 0, kernel.data(), kernel.size());
            a->pushToDevice();
        }
        rt.initialize();
        const double initialised = sinceStart();
        // a file holds either the whole array or one batch's worth, which is then replicated
        auto load = [&](Runtime::ArrayBase *a, const std::string &file) {
            if(a->getType() == Type::Double && file.size() > 4 && file.compare(file.size() - 4, 4, ".f32") == 0) {
                const auto values = readFile<float>(in + "/" + file);
                if(values.empty() || (a->getCount() % values.size()) != 0) { throw std::runtime_error(file + ": does not tile the array"); }
                for(size_t o = 0; o < a->getCount(); o += values.size()) { storeScalars(a, o, values.data(), values.size()); }
                return;
            }
            const auto bytes = readFile<char>(in + "/" + file);
            if(bytes.empty() || (a->getSizeBytes() % bytes.size()) != 0) {
                throw std::runtime_error(file + ": " + std::to_string(bytes.size()) + " bytes do not tile an array of " + std::to_string(a->getSizeBytes()));
            }
            for(size_t o = 0; o < a->getSizeBytes(); o += bytes.size()) {
                std::copy(bytes.begin(), bytes.end(), reinterpret_cast<char*>(a->getHostPointer()) + o);
            }
        };
        for(auto &p : pops) {
            if(p.model == "lif") { load(rt.getArray(*p.ng, "V"), p.name + ".V.f32"); load(rt.getArray(*p.ng, "RefracTime"), p.name + ".RefracTime.f32"); }
            else if(p.model == "lifa") {
                load(rt.getArray(*p.ng, "V"), p.name + ".V.f32"); load(rt.getArray(*p.ng, "RefracTime"), p.name + ".RefracTime.f32"); load(rt.getArray(*p.ng, "A"), p.name + ".A.f32");
            }
            else if(p.model == "izh") { load(rt.getArray(*p.ng, "V"), p.name + ".V.f32"); load(rt.getArray(*p.ng, "U"), p.name + ".U.f32"); }
            else if(p.model == "poisson") { load(rt.getArray(*p.ng, "timeStepToSpike"), p.name + ".timeStepToSpike.f32"); }
            else if(p.model == "ssa") {
                load(rt.getArray(*p.ng, "startSpike"), p.name + ".startSpike.u32");
                load(rt.getArray(*p.ng, "endSpike"), p.name + ".endSpike.u32");
                const auto st = readFile<float>(in + "/" + p.name + ".spikeTimes.f32");
                rt.allocateArray(*p.ng, "spikeTimes", st.size());
                auto *a = rt.getArray(*p.ng, "spikeTimes");
                storeScalars(a, 0, st.data(), st.size());
                a->pushToDevice();
            }
        }
        std::map<std::string, std::vector<float>> noise;
        for(auto &c : css) {
            if(c.model == "noise") {
                const unsigned int n = popByName.at(c.pop)->n;
                noise[c.name] = readFile<float>(in + "/" + c.name + ".noise.f32", (size_t)n * steps);
                rt.allocateArray(*c.cs, "noise", n);
            }
        }
        // per-synapse arrays are stored with the netspec's row stride; the backend may use a larger one
        auto backendStride = [&](const SynSpec &s) { return backend.getSynapticMatrixRowStride(*static_cast<const SynapseGroupInternal*>(s.sg)); };
        auto loadRows = [&](Runtime::ArrayBase *a, const std::string &file, const SynSpec &s, auto zero) {
            using T = decltype(zero);
            const size_t numPre = popByName.at(s.src)->n, stride = backendStride(s);
            const auto rows = readFile<T>(in + "/" + file, numPre * s.rowStride);
            // (variables a learning rule writes have one copy per batch: every copy starts from the file's values)
            const size_t copies = a->getCount() / (numPre * stride);
            if constexpr(std::is_same_v<T, float>) {
                for(size_t c = 0; c < copies; c++) {
                    for(size_t i = 0; i < numPre; i++) { storeScalars(a, (c * numPre + i) * stride, rows.data() + i * s.rowStride, s.rowStride); }
                }
            }
            else {
                auto *dst = a->getHostPointer<T>();
                for(size_t c = 0; c < copies; c++) {
                    for(size_t i = 0; i < numPre; i++) { std::copy_n(rows.begin() + i * s.rowStride, s.rowStride, dst + (c * numPre + i) * stride); }
                }
            }
        };
        for(auto &s : syns) {
            if(s.matrix == "sparse") {
                load(rt.getArray(*s.sg, "rowLength"), s.name + ".rowLength.u32");
                loadRows(rt.getArray(*s.sg, "ind"), s.name + ".ind.u32", s, uint32_t(0));
                if(s.wum != "static_const") loadRows(rt.getArray(*s.sg, "g"), s.name + ".g.f32", s, float(0));
                if(s.wum == "static_delay") loadRows(rt.getArray(*s.sg, "d"), s.name + ".d.u8", s, uint8_t(0));
            }
            else if(s.matrix == "bitmask") {
                load(rt.getArray(*s.sg, "gp"), s.name + ".gp.u32");
            }
            else if(s.wum != "static_const" && s.wum != "static_init" && s.wum != "static_kernel" && s.matrix != "procedural" && s.matrix != "sparse_init") {
                load(rt.getArray(*s.sg, "g"), s.name + ".g.f32");
            }
            if(s.wum == "stdp_trace") {
                rt.getArray(*s.sg, "preTrace")->memsetHostPointer(0);
                rt.getArray(*s.sg, "postTrace")->memsetHostPointer(0);
            }
        }
        rt.initializeSparse();
        for(auto &p : pops) {
            if(p.model != "lif_init") { continue; }
            auto *v = rt.getArray(*p.ng, "V"); v->pullFromDevice();
            appendScalars(out + "/" + p.name + ".V0.f32", v, 0, (size_t)p.n * batch);
        }
        // (how long a model takes from loading its code to its first step: allocation, initialize(), initializeSparse())
        {
            // (VmHWM of this process image: getrusage's ru_maxrss also carries the peak of the process that started this one)
            long peakKiB = 0;
            std::ifstream status("/proc/self/status");
            for(std::string line; std::getline(status, line); ) {
                if(line.rfind("VmHWM:", 0) == 0) { peakKiB = std::stol(line.substr(6)); }
            }
            std::cout << "ref_driver: ready after " << sinceStart() << " s (allocate " << allocated << ", initialize " << (initialised - allocated)
                      << "), peak resident host memory " << peakKiB / 1024 << " MiB" << std::endl;
        }
        // matrices initialised by snippets: what the initialisation produced, with the backend's row stride
        for(auto &s : syns) {
            if(s.matrix == "dense_init" || (s.matrix == "conv2d" && s.wum == "static_init")) {
                auto *g = rt.getArray(*s.sg, "g"); g->pullFromDevice();
                appendScalars(out + "/" + s.name + ".g.f32", g, 0, g->getCount());
                continue;
            }
            if((s.matrix != "sparse_init" && s.matrix != "conv2d_sparse") || deviceArrays) { continue; }
            const size_t numPre = popByName.at(s.src)->n, stride = backendStride(s);
            std::ofstream(out + "/" + s.name + ".rowStride.txt") << stride << std::endl;
            auto *rl = rt.getArray(*s.sg, "rowLength"); rl->pullFromDevice();
            auto *ind = rt.getArray(*s.sg, "ind"); ind->pullFromDevice();
            appendFile(out + "/" + s.name + ".rowLength.u32", rl->getHostPointer<uint32_t>(), numPre);
            appendFile(out + "/" + s.name + ".ind.u32", ind->getHostPointer<uint32_t>(), numPre * stride);
            if(s.wum != "static_const") {
                auto *g = rt.getArray(*s.sg, "g"); g->pullFromDevice();
                appendScalars(out + "/" + s.name + ".g.f32", g, 0, numPre * stride);
            }
        }

        // fuse map + remap dump
        {
            std::ofstream fm(out + "/fusemap.txt");
            for(auto &s : syns) {
                const auto *sgi = static_cast<const SynapseGroupInternal*>(s.sg);
                fm << s.name << " " << sgi->getFusedPSTarget().getName() << std::endl;
                if(s.wum == "stdp_trace" || s.wum == "stdp" || s.wum == "timing_copy" || s.wum == "prev_timing" || s.wum == "post_event") {
                    auto *cl = rt.getArray(*s.sg, "colLength"); auto *rm = rt.getArray(*s.sg, "remap");
                    cl->pullFromDevice(); rm->pullFromDevice();
                    appendFile(out + "/" + s.name + ".colLength.u32", cl->getHostPointer<uint32_t>(), cl->getCount());
                    // synapse indices are written in terms of the netspec's row stride
                    std::vector<uint32_t> remap(rm->getHostPointer<uint32_t>(), rm->getHostPointer<uint32_t>() + rm->getCount());
                    const uint32_t stride = (uint32_t)backendStride(s);
                    for(auto &r : remap) { r = (r / stride) * s.rowStride + (r % stride); }
                    appendFile(out + "/" + s.name + ".remap.u32", remap.data(), remap.size());
                    std::ofstream(out + "/" + s.name + ".colStride.txt") << sgi->getMaxSourceConnections() << std::endl;
                }
            }
        }

        auto pulled = [](Runtime::ArrayBase *a) { a->pullFromDevice(); return a; };
        auto snapshot = [&]() {
            for(auto &p : pops) {
                if(p.model == "ssa" || p.model == "poisson") continue;
                pulled(rt.getArray(*p.ng, "V"));
                pulled(rt.getArray(*p.ng, (p.model == "lif" || p.model == "lifa" || p.model == "lif_init") ? "RefracTime" : "U"));
                appendScalars(out + "/" + p.name + ".V.f32", rt.getArray(*p.ng, "V"), 0, (size_t)p.n * batch);
                if(p.model == "lif" || p.model == "lifa" || p.model == "lif_init") appendScalars(out + "/" + p.name + ".RefracTime.f32", rt.getArray(*p.ng, "RefracTime"), 0, (size_t)p.n * batch);
                if(p.model == "lifa") { auto *a = pulled(rt.getArray(*p.ng, "A")); appendScalars(out + "/" + p.name + ".A.f32", a, 0, (size_t)p.n * batch); }
                if(p.model == "izh") appendScalars(out + "/" + p.name + ".U.f32", rt.getArray(*p.ng, "U"), 0, (size_t)p.n * batch);
            }
            for(auto &s : syns) {
                const auto *sgi = static_cast<const SynapseGroupInternal*>(s.sg);
                if(&sgi->getFusedPSTarget() == sgi) {
                    auto *a = pulled(rt.getArray(*s.sg, "outPost"));
                    appendScalars(out + "/" + s.name + ".outPost.f32", a, 0, a->getCount());
                    if(sgi->isDendriticOutputDelayRequired()) {
                        auto *d = pulled(rt.getArray(*s.sg, "denDelay"));
                        appendScalars(out + "/" + s.name + ".denDelay.f32", d, 0, d->getCount());
                    }
                }
                if(s.wum == "stdp_trace" || s.wum == "stdp") {
                    auto *a = pulled(rt.getArray(*s.sg, "g"));
                    const size_t numPre = popByName.at(s.src)->n, stride = backendStride(s);
                    for(size_t i = 0; i < numPre * batch; i++) { appendScalars(out + "/" + s.name + ".g.f32", a, i * stride, s.rowStride); }
                }
                if(s.wum == "post_event") {
                    const size_t numPre = popByName.at(s.src)->n, stride = backendStride(s);
                    auto *a = pulled(rt.getArray(*s.sg, "hits"));
                    for(size_t i = 0; i < numPre * batch; i++) { appendScalars(out + "/" + s.name + ".hits.f32", a, i * stride, s.rowStride); }
                }
                if(s.wum == "leaky_graded") {
                    const size_t numPre = popByName.at(s.src)->n, stride = backendStride(s);
                    auto *a = pulled(rt.getArray(*s.sg, "x"));
                    for(size_t i = 0; i < numPre * batch; i++) { appendScalars(out + "/" + s.name + ".x.f32", a, i * stride, s.rowStride); }
                }
                if(s.wum == "timing_copy" || s.wum == "prev_timing") {
                    const size_t numPre = popByName.at(s.src)->n, stride = backendStride(s);
                    for(const char *var : {"wPre", "wPost"}) {
                        auto *a = pulled(rt.getArray(*s.sg, var));
                        for(size_t i = 0; i < numPre * batch; i++) { appendScalars(out + "/" + s.name + "." + var + ".f32", a, i * stride, s.rowStride); }
                    }
                }
                if(s.wum == "timing_copy") {
                    for(const char *var : {"sPre", "sPost"}) {
                        auto *a = pulled(rt.getArray(*s.sg, var));
                        appendScalars(out + "/" + s.name + "." + var + ".f32", a, 0, a->getCount());
                    }
                }
                if(s.wum == "stdp_trace") {
                    auto *a = pulled(rt.getArray(*s.sg, "preTrace")); auto *b = pulled(rt.getArray(*s.sg, "postTrace"));
                    appendScalars(out + "/" + s.name + ".preTrace.f32", a, 0, a->getCount());
                    appendScalars(out + "/" + s.name + ".postTrace.f32", b, 0, b->getCount());
                }
            }
        };

        // variables of the custom updates, and what they write in the projections they refer to (per-synapse arrays row by
        // row in terms of the netspec's stride, like the projections' own)
        auto dumpRows = [&](Runtime::ArrayBase *a, const std::string &file, const SynSpec &q) {
            a->pullFromDevice();
            if(q.matrix == "sparse") {
                const size_t numPre = popByName.at(q.src)->n, stride = backendStride(q), copies = a->getCount() / (numPre * stride);
                for(size_t i = 0; i < numPre * copies; i++) { appendScalars(out + "/" + file, a, i * stride, q.rowStride); }
            }
            else {
                appendScalars(out + "/" + file, a, 0, a->getCount());
            }
        };
        auto customSnapshot = [&]() {
            for(auto &c : customs) {
                if(c.kind == "decay") {
                    auto *a = pulled(rt.getArray(*c.cu, "applied"));
                    appendScalars(out + "/" + c.name + ".applied.f32", a, 0, a->getCount());
                }
                else if(c.kind == "neuron_reduce") {
                    for(const char *var : {"sum", "peak"}) {
                        auto *a = pulled(rt.getArray(*c.cu, var));
                        appendScalars(out + "/" + c.name + "." + var + ".f32", a, 0, a->getCount());
                    }
                }
                else if(c.kind == "wu_decay") {
                    const SynSpec &q = *synByName.at(c.target);
                    dumpRows(rt.getArray(*c.cuWU, "total"), c.name + ".total.f32", q);
                    dumpRows(rt.getArray(*c.cuWU, "when"), c.name + ".when.f32", q);
                    dumpRows(rt.getArray(*q.sg, "g"), c.name + ".w.f32", q);
                }
                else if(c.kind == "batch_reduce") {
                    const SynSpec &q = *synByName.at(c.target);
                    dumpRows(rt.getArray(*c.cuWU, "sum"), c.name + ".sum.f32", q);
                    dumpRows(rt.getArray(*c.cuWU, "peak"), c.name + ".peak.f32", q);
                    dumpRows(rt.getArray(*q.sg, "g"), c.name + ".w.f32", q);
                }
                else if(c.kind == "transpose") {
                    dumpRows(rt.getArray(*synByName.at(c.target2)->sg, "g"), c.name + ".transposed.f32", *synByName.at(c.target2));
                }
                else if(c.kind == "prune" || c.kind == "sprout") {
                    // the rewired matrix: row lengths, and targets and weights row by row in terms of the netspec's stride
                    const SynSpec &q = *synByName.at(c.target);
                    const size_t numPre = popByName.at(q.src)->n, stride = backendStride(q);
                    auto *rl = pulled(rt.getArray(*q.sg, "rowLength")); auto *ind = pulled(rt.getArray(*q.sg, "ind"));
                    appendFile(out + "/" + c.name + ".rowLength.u32", rl->getHostPointer<uint32_t>(), numPre);
                    for(size_t i = 0; i < numPre; i++) { appendFile(out + "/" + c.name + ".ind.u32", ind->getHostPointer<uint32_t>() + i * stride, q.rowStride); }
                    dumpRows(rt.getArray(*q.sg, "g"), c.name + ".w.f32", q);
                    if(c.kind == "prune") {
                        auto *a = pulled(rt.getArray(*c.ccu, "removed"));
                        appendScalars(out + "/" + c.name + ".removed.f32", a, 0, a->getCount());
                    }
                    else {
                        dumpRows(rt.getArray(*c.ccu, "born"), c.name + ".born.f32", q);
                        auto *a = pulled(rt.getArray(*c.ccu, "next"));
                        appendFile(out + "/" + c.name + ".next.u32", a->getHostPointer<uint32_t>(), a->getCount());
                    }
                }
            }
        };

        const auto loopStart = std::chrono::steady_clock::now();
        double firstSeconds = 0.0;
        for(unsigned int i = 0; i < steps; i++) {
            for(auto &c : css) {
                if(c.model == "noise") {
                    const unsigned int n = popByName.at(c.pop)->n;
                    auto *a = rt.getArray(*c.cs, "noise");
                    storeScalars(a, 0, noise[c.name].data() + (size_t)i * n, n);
                    a->pushToDevice();
                }
            }
            // scheduled parameter changes (Runtime::setDynamicParamValue, runtime.cc:945-976): in force from step d.step on
            for(const auto &d : dynamics) {
                if(d.step != i) { continue; }
                const Type::NumericValue value(d.value);
                if(d.kind == "neuron") { rt.setDynamicParamValue(*popByName.at(d.group)->ng, d.param, value); }
                else if(d.kind == "cs") { for(auto &c : css) { if(c.name == d.group) { rt.setDynamicParamValue(*c.cs, d.param, value); } } }
                else { for(auto &q : syns) { if(q.name == d.group) { rt.setDynamicParamValue(*q.sg, d.param, value); } } }
            }
            rt.stepTime();
            for(const auto &c : customCalls) { if(((i + 1) % c.every) == 0) { rt.customUpdate(c.group); } }
            if(snap && ((i + 1) % snap) == 0) { snapshot(); customSnapshot(); }
            // the first call also builds whatever the backend prepares lazily (the MI355X backend: its device tables)
            if(i == 0) { firstSeconds = std::chrono::duration<double>(std::chrono::steady_clock::now() - loopStart).count(); }
        }
        // a blocking pull drains whatever the backend still has queued, so the loop time below is complete
        for(auto &p : pops) { if(p.model != "ssa" && p.model != "poisson") { rt.getArray(*p.ng, "V")->pullFromDevice(); break; } }
        const double loopSeconds = std::chrono::duration<double>(std::chrono::steady_clock::now() - loopStart).count();
        std::cout << "ref_driver: stepping loop " << loopSeconds << " s for " << steps << " steps ("
                  << loopSeconds / steps * 1e6 << " us per Runtime::stepTime, snapshots included; first call " << firstSeconds * 1e3
                  << " ms, the others " << (steps > 1 ? (loopSeconds - firstSeconds) / (steps - 1) * 1e6 : 0.0) << " us each)" << std::endl;
        if(!snap || (steps % snap) != 0) { snapshot(); customSnapshot(); }

        // spike rasters as (step, id) pairs; the reference reports times in ms = step*dt
        rt.pullRecordingBuffersFromDevice();
        for(auto &p : pops) {
            const auto ev = rt.getRecordedSpikes(*p.ng);
            // the reference's decode lists the ids of one timestep in bit-scan order; sort them.
            // One file per batch: <pop>.spikes.u32 for batch 0, <pop>.spikes.b<k>.u32 for the others
            for(unsigned int bi = 0; bi < batch; bi++) {
                std::vector<std::pair<uint32_t, uint32_t>> sorted;
                const auto &times = ev.at(bi).first; const auto &ids = ev.at(bi).second;
                for(size_t k = 0; k < times.size(); k++) {
                    sorted.emplace_back((uint32_t)std::llround(times[k] / dt), ids[k]);
                }
                std::sort(sorted.begin(), sorted.end());
                std::vector<uint32_t> pairs;
                for(const auto &s : sorted) { pairs.push_back(s.first); pairs.push_back(s.second); }
                appendFile(out + "/" + p.name + ".spikes" + (bi ? ".b" + std::to_string(bi) : std::string()) + ".u32", pairs.data(), pairs.size());
            }
        }
        // recorded spike-like events of the graded projections, as (step, presynaptic id) pairs of batch 0
        for(auto &s : syns) {
            if(s.wum != "static_graded") continue;
            const auto ev = rt.getRecordedPreSpikeEvents(*s.sg);
            std::vector<std::pair<uint32_t, uint32_t>> sorted;
            const auto &times = ev.at(0).first; const auto &ids = ev.at(0).second;
            for(size_t k = 0; k < times.size(); k++) { sorted.emplace_back((uint32_t)std::llround(times[k] / dt), ids[k]); }
            std::sort(sorted.begin(), sorted.end());
            std::vector<uint32_t> pairs;
            for(const auto &e : sorted) { pairs.push_back(e.first); pairs.push_back(e.second); }
            appendFile(out + "/" + s.name + ".events.u32", pairs.data(), pairs.size());
        }
        if(timing) {
            std::cout << "ref_driver: timers init " << rt.getInitTime() << " initSparse " << rt.getInitSparseTime() << " neuronUpdate " << rt.getNeuronUpdateTime()
                      << " presynapticUpdate " << rt.getPresynapticUpdateTime() << " postsynapticUpdate " << rt.getPostsynapticUpdateTime() << std::endl;
            for(const auto &c : customCalls) {
                std::cout << "ref_driver: timers customUpdate " << c.group << " " << rt.getCustomUpdateTime(c.group) << " transpose " << rt.getCustomUpdateTransposeTime(c.group) << std::endl;
            }
        }
        std::cout << "ref_driver: " << name << " ran " << steps << " steps" << std::endl;
    }
    catch(const std::exception &e) {
        std::cerr << "ref_driver error: " << e.what() << std::endl;
        return 1;
    }
    return 0;
}
