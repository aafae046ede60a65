// GeNN::CodeGenerator::MI355X::Backend (see backend.h for the division of labour).
#include "backend.h"
#include "optimiser.h"

#include <sys/mman.h>
#include <algorithm>
#include <cctype>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <sstream>
#include <stdexcept>

#include "currentSourceModels.h"
#include "gennUtils.h"
#include "initToeplitzConnectivitySnippet.h"
#include "logging.h"
#include "neuronModels.h"
#include "postsynapticModels.h"
#include "weightUpdateModels.h"

#include "code_generator/codeGenUtils.h"
#include "code_generator/codeStream.h"
#include "code_generator/modelSpecMerged.h"
#include "code_generator/standardLibrary.h"
#include "runtime/runtime.h"

#include "genn_mi355x.h"

using namespace GeNN;
using namespace GeNN::CodeGenerator;

namespace
{
void check(int rc, const char *what)
{
    if(rc != GENNMI_OK) {
        throw std::runtime_error(std::string("MI355X backend: ") + what + ": " + gennmi_last_error());
    }
}

[[noreturn]] void unsupported(const std::string &what)
{
    throw std::runtime_error("MI355X backend: " + what + " is not among the models the device library implements");
}

//--------------------------------------------------------------------------
// Array: a host buffer (generated initialisation code and merged groups work on host pointers) mirrored by a device
// buffer; the pair is registered with the device library so generated code can translate pointers.  Counterpart of the
// Array classes of the reference's backends (hip/backend.cc:61-236).  An array the model places on the device only
// (VarLocation::DEVICE) gets no host memory there; here it gets address space that is committed only where host code
// touches it and given back after every upload (gennmi_register_device_array), so a 4 GB index array that the device
// generates never exists on the host.  Host sides of moderate size are pinned, and a zero-copy array (HOST_DEVICE_ZERO_COPY)
// is one piece of pinned memory that both sides address.
//--------------------------------------------------------------------------
class Array : public Runtime::ArrayBase
{
public:
    Array(const Type::ResolvedType &type, size_t count, VarLocation location, bool uninitialized)
    :   ArrayBase(type, count, location, uninitialized), m_Device(nullptr)
    {
        if(count > 0) {
            allocate(count);
        }
    }
    virtual ~Array()
    {
        if(getCount() > 0) {
            try { free(); } catch(...) {}
        }
    }

    virtual void allocate(size_t count) final
    {
        setCount(count);
        m_Reserved = !(getLocation() & VarLocationAttribute::HOST);
        m_ZeroCopy = !m_Reserved && (getLocation() & VarLocationAttribute::ZERO_COPY);
        // pinned host memory where copies recur (recording buffers, state a user pulls while the model runs); the largest arrays,
        // which are uploaded once, stay pageable: pinning gigabytes costs more than their one copy saves
        m_Pinned = m_ZeroCopy || (!m_Reserved && getSizeBytes() <= PINNED_LIMIT);
        std::byte *host = nullptr;
        if(m_Pinned) {
            void *p = nullptr, *mapped = nullptr;
            check(gennmi_host_malloc(&p, getSizeBytes(), m_ZeroCopy ? 1 : 0, &mapped), "pinned host allocation");
            host = static_cast<std::byte*>(p);
            if(m_ZeroCopy) {
                setHostPointer(host);
                m_Device = mapped;
                check(gennmi_register_mirror(host, m_Device, getSizeBytes()), "array registration");
                return;
            }
        }
        else if(m_Reserved) {
            void *space = mmap(nullptr, getSizeBytes(), PROT_READ | PROT_WRITE, MAP_PRIVATE | MAP_ANONYMOUS | MAP_NORESERVE, -1, 0);
            if(space == MAP_FAILED) { throw std::bad_alloc(); }
            host = static_cast<std::byte*>(space);
        }
        else {
            host = static_cast<std::byte*>(std::calloc(getSizeBytes(), 1));
            if(!host) { throw std::bad_alloc(); }
        }
        setHostPointer(host);
        check(gennmi_malloc(&m_Device, getSizeBytes()), "array allocation");
        check(gennmi_memset(m_Device, 0, getSizeBytes()), "array clear");
        check(m_Reserved ? gennmi_register_device_array(host, m_Device, getSizeBytes())
                         : gennmi_register_mirror(host, m_Device, getSizeBytes()), "array registration");
    }
    virtual void free() final
    {
        check(gennmi_unregister_mirror(getHostPointer()), "array deregistration");
        if(!m_ZeroCopy) { check(gennmi_free(m_Device), "array release"); }
        if(m_Pinned) { check(gennmi_host_free(getHostPointer()), "pinned host release"); }
        else if(m_Reserved) { munmap(getHostPointer(), getSizeBytes()); }
        else { std::free(getHostPointer()); }
        m_Device = nullptr;
        setHostPointer(nullptr);
        setCount(0);
    }
    virtual void pushToDevice() final { pushSlice1DToDevice(0, getCount()); }
    virtual void pullFromDevice() final { pullSlice1DFromDevice(0, getCount()); }
    virtual void pushSlice1DToDevice(size_t offset, size_t count) final
    {
        const auto [o, b] = slice(offset, count);
        if(m_ZeroCopy) { return; }          // one memory: nothing to copy (hip/backend.cc:131-136)
        check(gennmi_memcpy_to_device(static_cast<char*>(m_Device) + o, getHostPointer() + o, b), "push");
    }
    virtual void pullSlice1DFromDevice(size_t offset, size_t count) final
    {
        const auto [o, b] = slice(offset, count);
        if(m_ZeroCopy) {
            // one memory: what the device wrote is there once the steps still queued have run
            check(gennmi_synchronize(), "pull");
            return;
        }
        check(gennmi_memcpy_from_device(getHostPointer() + o, static_cast<const char*>(m_Device) + o, b), "pull");
    }
    virtual void memsetDeviceObject(int value) final
    {
        check(gennmi_memset(m_Device, value, getSizeBytes()), "memset");
    }
    virtual void serialiseDeviceObject(std::vector<std::byte> &bytes, bool pointerToPointer) const final
    {
        std::byte raw[sizeof(void*)];
        if(pointerToPointer) {
            void* const *pp = &m_Device;
            std::memcpy(raw, &pp, sizeof(void*));
        }
        else {
            std::memcpy(raw, &m_Device, sizeof(void*));
        }
        bytes.insert(bytes.end(), std::begin(raw), std::end(raw));
    }
    virtual void serialiseHostObject(std::vector<std::byte>&, bool) const final
    {
        throw std::runtime_error("MI355X arrays have no host objects");
    }

private:
    std::pair<size_t, size_t> slice(size_t offset, size_t count) const
    {
        if(offset + count > getCount()) {
            throw std::runtime_error("Slice overflows array");
        }
        const size_t elem = getType().getValue().size;
        return {offset * elem, count * elem};
    }

    static constexpr size_t PINNED_LIMIT = 64u << 20;
    void *m_Device;
    bool m_Reserved = false;    // the host side is address space without memory behind it (device-only array)
    bool m_Pinned = false;      // the host side is pinned memory
    bool m_ZeroCopy = false;    // ... mapped into the device's address space: host and device side are one memory
};

//--------------------------------------------------------------------------
// Model recognition: code strings are compared with all whitespace removed
//--------------------------------------------------------------------------
std::string squeeze(const std::string &code)
{
    std::string out;
    for(char c : code) {
        if(!std::isspace(static_cast<unsigned char>(c))) { out += c; }
    }
    return out;
}
bool same(const std::string &a, const std::string &b) { return squeeze(a) == squeeze(b); }

unsigned int recogniseNeuron(const NeuronModels::Base *m, const std::string &name)
{
    for(const auto &[builtin, id] : {std::pair<const NeuronModels::Base*, unsigned int>{NeuronModels::LIF::getInstance(), GENNMI_NEURON_LIF},
                                    {NeuronModels::Izhikevich::getInstance(), GENNMI_NEURON_IZHIKEVICH},
                                    {NeuronModels::SpikeSourceArray::getInstance(), GENNMI_NEURON_SPIKE_SOURCE_ARRAY}}) {
        if(m == builtin || (same(m->getSimCode(), builtin->getSimCode()) && same(m->getThresholdConditionCode(), builtin->getThresholdConditionCode())
                            && same(m->getResetCode(), builtin->getResetCode()))) {
            return id;
        }
    }
    unsupported("neuron model of population '" + name + "'");
}
unsigned int recognisePSM(const PostsynapticModels::Base *m, const std::string &name)
{
    if(same(m->getSimCode(), PostsynapticModels::ExpCurr::getInstance()->getSimCode())) { return GENNMI_PSM_EXPCURR; }
    if(same(m->getSimCode(), PostsynapticModels::DeltaCurr::getInstance()->getSimCode())) { return GENNMI_PSM_DELTACURR; }
    unsupported("postsynaptic model of projection '" + name + "'");
}
// pair-based additive STDP with all-to-all traces, as in the weight-update example of pygenn/genn_model.py:1448-1476
bool isTraceSTDP(const WeightUpdateModels::Base *m)
{
    return same(m->getPreSpikeSynCode(), "addToPost(g); const scalar dt = t - st_post; if(dt > 0) { const scalar newWeight = g - (aMinus * postTrace); g = fmin(wMax, fmax(wMin, newWeight)); }")
        && same(m->getPostSpikeSynCode(), "const scalar dt = t - st_pre; if(dt > 0) { const scalar newWeight = g + (aPlus * preTrace); g = fmin(wMax, fmax(wMin, newWeight)); }")
        && same(m->getPreSpikeCode(), "preTrace += 1.0;") && same(m->getPostSpikeCode(), "postTrace += 1.0;")
        && same(m->getPreDynamicsCode(), "preTrace *= tauPlusDecay;") && same(m->getPostDynamicsCode(), "postTrace *= tauMinusDecay;")
        && m->getSynapseDynamicsCode().empty() && m->getPreEventSynCode().empty() && m->getPostEventSynCode().empty();
}
// the built-in additive STDP with nearest-neighbour pairing (weightUpdateModels.h:345-367)
bool isAdditiveSTDP(const WeightUpdateModels::Base *m)
{
    const auto *builtin = WeightUpdateModels::STDP::getInstance();
    return same(m->getPreSpikeSynCode(), builtin->getPreSpikeSynCode()) && same(m->getPostSpikeSynCode(), builtin->getPostSpikeSynCode())
        && m->getPreSpikeCode().empty() && m->getPostSpikeCode().empty() && m->getPreDynamicsCode().empty() && m->getPostDynamicsCode().empty()
        && m->getSynapseDynamicsCode().empty() && m->getPreEventSynCode().empty() && m->getPostEventSynCode().empty()
        && m->getVars().size() == 1 && m->getVars()[0].name == "g" && m->getParams().size() == 6 && m->getPreVars().empty() && m->getPostVars().empty();
}
// StaticGraded (weightUpdateModels.h:308-319): spike-like events while V > Epre, each adding
// fmax(0, g * tanh((V_pre - Epre) / Vslope) * dt).  The built-in's event code spells the presynaptic potential `V_pre`;
// a model with the same code that spells it `V` — the name the 5.4.0 generator gives a presynaptic neuron variable
// reference in synapse code — is the same model.
bool isStaticGraded(const WeightUpdateModels::Base *m)
{
    const auto *builtin = WeightUpdateModels::StaticGraded::getInstance();
    auto respelt = [](std::string code)
    {
        for(size_t at = code.find("V_pre"); at != std::string::npos; at = code.find("V_pre", at)) { code.replace(at, 5, "V"); }
        return code;
    };
    const bool onlyEvents = m->getPreSpikeSynCode().empty() && m->getPostSpikeSynCode().empty() && m->getSynapseDynamicsCode().empty()
                            && m->getPostEventSynCode().empty() && m->getPreSpikeCode().empty() && m->getPostSpikeCode().empty()
                            && m->getPreDynamicsCode().empty() && m->getPostDynamicsCode().empty() && m->getPostEventThresholdConditionCode().empty();
    const auto refs = m->getPreNeuronVarRefs();
    return onlyEvents && same(m->getPreEventThresholdConditionCode(), builtin->getPreEventThresholdConditionCode())
           && (same(m->getPreEventSynCode(), builtin->getPreEventSynCode()) || same(m->getPreEventSynCode(), respelt(builtin->getPreEventSynCode())))
           && m->getVars().size() == 1 && m->getVars()[0].name == "g" && refs.size() == 1 && refs[0].name == "V"
           && m->getParams().size() == 2 && m->getPreVars().empty() && m->getPostVars().empty();
}

unsigned int recogniseWUM(const WeightUpdateModels::Base *m, const std::string &name)
{
    const bool plain = m->getPostSpikeSynCode().empty() && m->getSynapseDynamicsCode().empty() && m->getPreEventSynCode().empty()
                       && m->getPostEventSynCode().empty() && m->getPreSpikeCode().empty() && m->getPostSpikeCode().empty()
                       && m->getPreDynamicsCode().empty() && m->getPostDynamicsCode().empty();
    if(plain && same(m->getPreSpikeSynCode(), WeightUpdateModels::StaticPulse::getInstance()->getPreSpikeSynCode())
       && m->getVars().size() == 1) { return GENNMI_WUM_STATIC_PULSE; }
    // StaticPulseConstantWeight (weightUpdateModels.h:202-213): the same code with g a parameter instead of a variable
    if(plain && same(m->getPreSpikeSynCode(), WeightUpdateModels::StaticPulseConstantWeight::getInstance()->getPreSpikeSynCode())
       && m->getVars().empty() && m->getParams().size() == 1 && m->getParams()[0].name == "g") { return GENNMI_WUM_STATIC_PULSE_CONSTANT_WEIGHT; }
    if(plain && same(m->getPreSpikeSynCode(), WeightUpdateModels::StaticPulseDendriticDelay::getInstance()->getPreSpikeSynCode())) {
        return GENNMI_WUM_STATIC_PULSE_DENDRITIC_DELAY;
    }
    if(isTraceSTDP(m)) { return GENNMI_WUM_STDP_TRACE; }
    if(isAdditiveSTDP(m)) { return GENNMI_WUM_STDP; }
    if(isStaticGraded(m)) { return GENNMI_WUM_STATIC_GRADED; }
    // presynaptic output: the static_pulse_reverse model of the reference's tests/features/test_event_propagation.py:584-590
    if(plain && same(m->getPreSpikeSynCode(), "addToPre(g);") && m->getVars().size() == 1 && m->getVars()[0].name == "g") { return GENNMI_WUM_STATIC_PULSE_REVERSE; }
    unsupported("weight update model of projection '" + name + "'");
}

//--------------------------------------------------------------------------
// Constants in generated code.  The reference prints a parameter that is equal in every group of a merged group as
// a literal of the model's scalar type and passes a differing one through a struct field of that type
// (environment.h:483-511); both are reproduced so device arithmetic sees the same fp32 values.
//--------------------------------------------------------------------------
std::string table(const std::vector<Type::NumericValue> &values, const Type::ResolvedType &type)
{
    const bool uniform = std::all_of(values.cbegin(), values.cend(), [&](const auto &v){ return v == values.front(); });
    std::ostringstream os;
    os << "{";
    for(size_t i = 0; i < values.size(); i++) {
        if(uniform) {
            os << Type::writeNumeric(values[i], type);
        }
        else {
            char buf[64];
            std::snprintf(buf, sizeof(buf), "%a", values[i].cast<double>());
            os << "(" << type.getName() << ")" << buf;
        }
        os << ((i + 1 == values.size()) ? "" : ", ");
    }
    os << "}";
    return os.str();
}
std::string tableU32(const std::vector<uint64_t> &values)
{
    std::ostringstream os;
    os << "{";
    for(size_t i = 0; i < values.size(); i++) { os << values[i] << ((i + 1 == values.size()) ? "u" : "u, "); }
    os << "}";
    return os.str();
}
}   // anonymous namespace

//--------------------------------------------------------------------------
// GeNN::CodeGenerator::MI355X::Backend
//--------------------------------------------------------------------------
namespace GeNN::CodeGenerator::MI355X
{
Backend::Backend(const Preferences &preferences, bool generatedKernels, bool customUpdateKernels)
:   BackendBase(preferences), m_GeneratedKernels(generatedKernels), m_CustomUpdateKernels(customUpdateKernels && !generatedKernels)
{
}
//--------------------------------------------------------------------------
// updateNeurons: one descriptor per group of every merged neuron update group, built once by
// gennmiBuildNeuronGroups(); the call itself advances the whole timestep (see gennmi_step)
//--------------------------------------------------------------------------
void Backend::genNeuronUpdate(CodeStream &os, FileStreamCreator, ModelSpecMerged &modelMerged,
                              BackendBase::MemorySpaces &memorySpaces, HostHandler preambleHandler) const
{
    if(m_GeneratedKernels) {
        genNeuronUpdateGenerated(os, modelMerged, memorySpaces, preambleHandler);
        return;
    }
    const ModelSpecInternal &model = modelMerged.getModel();
    const unsigned int batchSize = model.getBatchSize();
    const auto scalar = model.getPrecision();
    if(scalar != Type::Float || model.getTimePrecision() != Type::Float) {
        throw std::runtime_error("MI355X backend: only single-precision models are supported");
    }

    std::ostringstream bodyStream;
    CodeStream body(bodyStream);
    EnvironmentLibrary libEnv(body, StandardLibrary::getMathsFunctions());

    // host-side advance of the spike-queue pointers of populations with axonal delay slots, run by updateNeurons()
    std::ostringstream queueStream;
    CodeStream queue(queueStream);

    body << "void gennmiBuildNeuronGroups()";
    {
        CodeStream::Scope b(body);
        EnvironmentExternal funcEnv(libEnv);
        modelMerged.genMergedNeuronUpdateGroups(
            *this, memorySpaces,
            [this, &funcEnv, &queue, &model, batchSize, scalar](auto &n)
            {
                const auto &arch = n.getArchetype();
                const size_t numGroups = n.getGroups().size();
                const unsigned int neuronModel = recogniseNeuron(arch.getModel(), arch.getName());
                // axonal delay slots: supported for populations whose spikes feed static projections only
                if(arch.isDelayRequired() && (arch.isSpikeTimeRequired() || !n.getMergedOutSynWUMPreCodeGroups().empty() || !n.getMergedInSynWUMPostCodeGroups().empty())) {
                    unsupported("delay slots together with plasticity on population '" + arch.getName() + "'");
                }
                // random numbers in the step: only the PoissonExp current source draws any (recognised below); the recognised
                // neuron and postsynaptic models draw none
                if(arch.isSimRNGRequired() && std::none_of(arch.getCurrentSources().cbegin(), arch.getCurrentSources().cend(),
                                                           [](const CurrentSourceInternal *cs){ return Utils::isRNGRequired(cs->getInjectionCodeTokens()); })) {
                    unsupported("random numbers in the update of population '" + arch.getName() + "'");
                }
                if(arch.isPrevSpikeTimeRequired()) { unsupported("previous spike times of population '" + arch.getName() + "'"); }
                if(n.getMergedSpikeEventGroups().size() > GENNMI_MAX_SPK_EVENT) { unsupported("more than 2 spike-like event conditions on population '" + arch.getName() + "'"); }
                if(!n.getMergedSpikeEventGroups().empty() && (arch.isDelayRequired() || arch.isSpikeEventTimeRequired() || arch.isPrevSpikeEventTimeRequired())) {
                    unsupported("delay slots or event times with spike-like events on population '" + arch.getName() + "'");
                }
                if(n.getMergedOutSynPreOutputGroups().size() > GENNMI_MAX_PRE_OUTPUT) { unsupported("more than 2 presynaptic outputs into population '" + arch.getName() + "'"); }

                // Parameters reach the device as constants of the descriptors built once, before the first step.  A parameter the
                // model marks dynamic (setParamDynamic: the reference gives it a DYNAMIC merged-struct field that
                // setDynamicParamValue rewrites at run time, neuronGroup.h:135, currentSource.h:67, synapseGroup.h:187) would
                // keep its first value for ever, so such a model is refused rather than run wrongly.
                for(const auto &g : n.getGroups()) {
                    for(const auto &p : g.get().getModel()->getParams()) {
                        if(g.get().isParamDynamic(p.name)) { unsupported("dynamic parameter '" + p.name + "' of population '" + g.get().getName() + "'"); }
                    }
                    for(const auto *cs : g.get().getCurrentSources()) {
                        for(const auto &p : cs->getModel()->getParams()) {
                            if(cs->isParamDynamic(p.name)) { unsupported("dynamic parameter '" + p.name + "' of current source '" + cs->getName() + "'"); }
                        }
                    }
                    for(const auto *sg : g.get().getFusedPSMInSyn()) {
                        for(const auto &p : sg->getPSInitialiser().getSnippet()->getParams()) {
                            if(sg->isPSParamDynamic(p.name)) { unsupported("dynamic postsynaptic-model parameter '" + p.name + "' of projection '" + sg->getName() + "'"); }
                        }
                    }
                }

                // values of one quantity across the groups of this merged group
                auto perGroup = [&n](auto fn)
                {
                    std::vector<Type::NumericValue> v;
                    for(const auto &g : n.getGroups()) { v.push_back(fn(g.get())); }
                    return v;
                };

                CodeStream::Scope b(funcEnv.getStream());
                funcEnv.getStream() << "// merged neuron update group " << n.getIndex() << std::endl;
                funcEnv.getStream() << "for(unsigned int g = 0; g < " << numGroups << "; g++)";
                CodeStream::Scope b2(funcEnv.getStream());
                funcEnv.getStream() << "const auto *group = &mergedNeuronUpdateGroup" << n.getIndex() << "[g];" << std::endl;
                EnvironmentGroupMergedField<NeuronUpdateGroupMerged> env(funcEnv, n);
                buildStandardEnvironment(env, batchSize);
                CodeStream &out = env.getStream();

                // pointer fields of the merged struct, added under the names the reference's own backends use
                auto var = [&env](const std::string &name, const Type::ResolvedType &type, bool dynamic = false)
                {
                    env.addField(type.createPointer(), "_mi_" + name, name,
                                 [name](const auto &runtime, const auto &g, size_t) { return runtime.getArray(g, name); },
                                 "", dynamic ? GroupMergedFieldType::DYNAMIC : GroupMergedFieldType::STANDARD);
                    return "gennmiDev(" + env["_mi_" + name] + ")";
                };

                out << "gennmi_neuron_update_group_t d = {};" << std::endl;
                out << "d.model = " << neuronModel << "u;" << std::endl;
                out << "static const uint32_t numNeurons[] = " << tableU32([&n]{ std::vector<uint64_t> v; for(const auto &g : n.getGroups()) { v.push_back(g.get().getNumNeurons()); } return v; }()) << ";" << std::endl;
                out << "d.numNeurons = numNeurons[g];" << std::endl;

                std::vector<std::string> paramNames;
                if(neuronModel == GENNMI_NEURON_LIF) {
                    out << "d.var0 = " << var("V", scalar) << "; d.var1 = " << var("RefracTime", scalar) << ";" << std::endl;
                    paramNames = {"Ioffset", "Rmembrane", "Vrest", "ExpTC", "Vthresh", "Vreset", "TauRefrac"};
                }
                else if(neuronModel == GENNMI_NEURON_IZHIKEVICH) {
                    out << "d.var0 = " << var("V", scalar) << "; d.var1 = " << var("U", scalar) << ";" << std::endl;
                    paramNames = {"a", "b", "c", "d"};
                }
                else {
                    out << "d.startSpike = " << var("startSpike", Type::Uint32) << "; d.endSpike = " << var("endSpike", Type::Uint32) << ";" << std::endl;
                    out << "d.spikeTimes = " << var("spikeTimes", scalar, true) << ";" << std::endl;
                }
                for(size_t k = 0; k < paramNames.size(); k++) {
                    const std::string &p = paramNames[k];
                    out << "{ static const float v[] = " << table(perGroup([&p](const NeuronGroupInternal &g)
                        {
                            const auto it = g.getParams().find(p);
                            return (it != g.getParams().end()) ? it->second : g.getDerivedParams().at(p);
                        }), scalar) << "; d.params[" << k << "] = v[g]; }" << std::endl;
                }

                // fused postsynaptic models, in the order the reference applies them
                const auto &psms = n.getMergedInSynPSMGroups();
                if(psms.size() > GENNMI_MAX_PSM) { unsupported("more than 8 postsynaptic models on population '" + arch.getName() + "'"); }
                out << "d.numPSM = " << psms.size() << "u;" << std::endl;
                for(size_t k = 0; k < psms.size(); k++) {
                    auto &child = const_cast<NeuronUpdateGroupMerged::InSynPSM&>(psms[k]);
                    const auto &sg = child.getArchetype();
                    const unsigned int kind = recognisePSM(sg.getPSInitialiser().getSnippet(), sg.getName());
                    if(sg.getPostTargetVar() != "Isyn") { unsupported("postsynaptic target variable '" + sg.getPostTargetVar() + "'"); }
                    const std::string sfx = "InSyn" + std::to_string(child.getIndex());
                    const std::string dst = "d.psm[" + std::to_string(k) + "]";
                    EnvironmentGroupMergedField<NeuronUpdateGroupMerged::InSynPSM, NeuronUpdateGroupMerged> penv(env, child, n);
                    auto childPtr = [&penv, &sfx](const std::string &name, const Type::ResolvedType &type)
                    {
                        penv.addField(type.createPointer(), "_mi_" + name, name + sfx,
                                      [name](const auto &runtime, const auto &g, size_t) { return runtime.getArray(g, name); });
                        return "gennmiDev(" + penv["_mi_" + name] + ")";
                    };
                    auto childValues = [&child](auto fn)
                    {
                        std::vector<Type::NumericValue> v;
                        for(const auto &g : child.getGroups()) { v.push_back(fn(g.get())); }
                        return v;
                    };
                    CodeStream &pout = penv.getStream();
                    pout << dst << ".outPost = " << childPtr("outPost", scalar) << "; " << dst << ".kind = " << kind << "u;" << std::endl;
                    if(sg.isDendriticOutputDelayRequired()) {
                        pout << dst << ".denDelay = " << childPtr("denDelay", scalar) << "; " << dst << ".denDelayPtr = " << childPtr("denDelayPtr", Type::Uint32) << ";" << std::endl;
                        pout << "{ static const uint32_t v[] = " << tableU32([&child]{ std::vector<uint64_t> v; for(const auto &g : child.getGroups()) { v.push_back(g.get().getMaxDendriticDelayTimesteps()); } return v; }())
                             << "; " << dst << ".maxDenDelay = v[g]; }" << std::endl;
                    }
                    if(kind == GENNMI_PSM_EXPCURR) {
                        for(const char *p : {"init", "expDecay"}) {
                            pout << "{ static const float v[] = " << table(childValues([p](const SynapseGroupInternal &g){ return g.getPSInitialiser().getDerivedParams().at(p); }), scalar)
                                 << "; " << dst << "." << p << " = v[g]; }" << std::endl;
                        }
                    }
                }

                // current sources
                const auto &css = n.getMergedCurrentSourceGroups();
                if(css.size() > GENNMI_MAX_CS) { unsupported("more than 4 current sources on population '" + arch.getName() + "'"); }
                out << "d.numCS = " << css.size() << "u;" << std::endl;
                for(size_t k = 0; k < css.size(); k++) {
                    auto &child = const_cast<NeuronUpdateGroupMerged::CurrentSource&>(css[k]);
                    const auto &cs = child.getArchetype();
                    const std::string dst = "d.cs[" + std::to_string(k) + "]";
                    if(cs.getTargetVar() != "Isyn") { unsupported("current source target variable '" + cs.getTargetVar() + "'"); }
                    EnvironmentGroupMergedField<NeuronUpdateGroupMerged::CurrentSource, NeuronUpdateGroupMerged> cenv(env, child, n);
                    CodeStream &cout = cenv.getStream();
                    if(same(cs.getModel()->getInjectionCode(), CurrentSourceModels::DC::getInstance()->getInjectionCode())) {
                        std::vector<Type::NumericValue> amps;
                        for(const auto &g : child.getGroups()) { amps.push_back(g.get().getParams().at("amp")); }
                        cout << "{ static const float v[] = " << table(amps, scalar) << "; " << dst << ".kind = " << GENNMI_CS_DC << "u; " << dst << ".amp = v[g]; }" << std::endl;
                    }
                    // one value per neuron read from an array the host refills before every step
                    else if(same(cs.getModel()->getInjectionCode(), "injectCurrent(noise[id]);") && cs.getModel()->getExtraGlobalParams().size() == 1) {
                        cenv.addField(scalar.createPointer(), "_mi_noise", "noiseCS" + std::to_string(child.getIndex()),
                                      [](const auto &runtime, const auto &g, size_t) { return runtime.getArray(g, "noise"); },
                                      "", GroupMergedFieldType::DYNAMIC);
                        cout << dst << ".kind = " << GENNMI_CS_ARRAY << "u; " << dst << ".arraySteps = 1u; " << dst << ".array = gennmiDev(" << cenv["_mi_noise"] << ");" << std::endl;
                    }
                    // PoissonExp: the uniforms of (neuron, step) are counter-based generator calls under the model's seed; one
                    // stream per source, numbered by its place in the model's (name-ordered) list of current sources
                    else if(same(cs.getModel()->getInjectionCode(), CurrentSourceModels::PoissonExp::getInstance()->getInjectionCode())) {
                        cenv.addField(scalar.createPointer(), "_mi_current", "currentCS" + std::to_string(child.getIndex()),
                                      [](const auto &runtime, const auto &g, size_t) { return runtime.getArray(g, "current"); });
                        cout << dst << ".kind = " << GENNMI_CS_POISSON_EXP << "u; " << dst << ".current = gennmiDev(" << cenv["_mi_current"] << "); "
                             << dst << ".seed = " << model.getSeed() << "ull;" << std::endl;
                        for(const auto &[field, param] : {std::pair<const char*, const char*>{"init", "Init"}, {"expDecay", "ExpDecay"}, {"expMinusLambda", "ExpMinusLambda"}}) {
                            std::vector<Type::NumericValue> values;
                            for(const auto &g : child.getGroups()) { values.push_back(g.get().getDerivedParams().at(param)); }
                            cout << "{ static const float v[] = " << table(values, scalar) << "; " << dst << "." << field << " = v[g]; }" << std::endl;
                        }
                        std::vector<uint64_t> streams;
                        for(const auto &g : child.getGroups()) {
                            streams.push_back(1000 + (uint64_t)std::distance(model.getLocalCurrentSources().cbegin(), model.getLocalCurrentSources().find(g.get().getName())));
                        }
                        cout << "{ static const uint32_t v[] = " << tableU32(streams) << "; " << dst << ".stream = v[g]; }" << std::endl;
                    }
                    else {
                        unsupported("current source model of '" + cs.getName() + "'");
                    }
                }

                // trace variables of plastic projections leaving / entering the population
                const auto &wuPre = n.getMergedOutSynWUMPreCodeGroups();
                const auto &wuPost = n.getMergedInSynWUMPostCodeGroups();
                if(wuPre.size() > 1 || wuPost.size() > 1) { unsupported("more than one plastic projection per side of population '" + arch.getName() + "'"); }
                if(!wuPre.empty()) {
                    auto &child = const_cast<NeuronUpdateGroupMerged::OutSynWUMPreCode&>(wuPre[0]);
                    if(!isTraceSTDP(child.getArchetype().getWUInitialiser().getSnippet())) { unsupported("presynaptic weight-update code of '" + child.getArchetype().getName() + "'"); }
                    EnvironmentGroupMergedField<NeuronUpdateGroupMerged::OutSynWUMPreCode, NeuronUpdateGroupMerged> wenv(env, child, n);
                    wenv.addField(scalar.createPointer(), "_mi_preTrace", "preTraceOutSynWUMPre" + std::to_string(child.getIndex()),
                                  [](const auto &runtime, const auto &g, size_t) { return runtime.getArray(g, "preTrace"); });
                    std::vector<Type::NumericValue> decay;
                    for(const auto &g : child.getGroups()) { decay.push_back(g.get().getWUInitialiser().getDerivedParams().at("tauPlusDecay")); }
                    wenv.getStream() << "{ static const float v[] = " << table(decay, scalar) << "; d.preTrace = gennmiDev(" << wenv["_mi_preTrace"] << "); d.preDecay = v[g]; }" << std::endl;
                }
                if(!wuPost.empty()) {
                    auto &child = const_cast<NeuronUpdateGroupMerged::InSynWUMPostCode&>(wuPost[0]);
                    if(!isTraceSTDP(child.getArchetype().getWUInitialiser().getSnippet())) { unsupported("postsynaptic weight-update code of '" + child.getArchetype().getName() + "'"); }
                    EnvironmentGroupMergedField<NeuronUpdateGroupMerged::InSynWUMPostCode, NeuronUpdateGroupMerged> wenv(env, child, n);
                    wenv.addField(scalar.createPointer(), "_mi_postTrace", "postTraceInSynWUMPost" + std::to_string(child.getIndex()),
                                  [](const auto &runtime, const auto &g, size_t) { return runtime.getArray(g, "postTrace"); });
                    std::vector<Type::NumericValue> decay;
                    for(const auto &g : child.getGroups()) { decay.push_back(g.get().getWUInitialiser().getDerivedParams().at("tauMinusDecay")); }
                    wenv.getStream() << "{ static const float v[] = " << table(decay, scalar) << "; d.postTrace = gennmiDev(" << wenv["_mi_postTrace"] << "); d.postDecay = v[g]; }" << std::endl;
                }

                // spike arrays: the first is the queue proper, the others receive copies
                const auto &spikes = n.getMergedSpikeGroups();
                if(spikes.size() > 1 + GENNMI_MAX_EXTRA_SPK) { unsupported("more than 4 spike arrays on population '" + arch.getName() + "'"); }
                for(size_t k = 0; k < spikes.size(); k++) {
                    auto &child = const_cast<NeuronUpdateGroupMerged::SynSpike&>(spikes[k]);
                    const std::string sfx = "SynSpike" + std::to_string(child.getIndex());
                    EnvironmentGroupMergedField<NeuronUpdateGroupMerged::SynSpike, NeuronUpdateGroupMerged> senv(env, child, n);
                    senv.addField(Type::Uint32.createPointer(), "_mi_spkCnt", "spkCnt" + sfx,
                                  [&n](const auto &runtime, const auto &g, size_t i) { return runtime.getFusedEventArray(n, i, g, "SpkCnt"); });
                    senv.addField(Type::Uint32.createPointer(), "_mi_spk", "spk" + sfx,
                                  [&n](const auto &runtime, const auto &g, size_t i) { return runtime.getFusedEventArray(n, i, g, "Spk"); });
                    const std::string cnt = "gennmiDev(" + senv["_mi_spkCnt"] + ")", spk = "gennmiDev(" + senv["_mi_spk"] + ")";
                    if(k == 0) {
                        senv.getStream() << "d.spkCnt = " << cnt << "; d.spk = " << spk << ";" << std::endl;
                    }
                    else {
                        senv.getStream() << "d.extraSpkCnt[" << (k - 1) << "] = " << cnt << "; d.extraSpk[" << (k - 1) << "] = " << spk << ";" << std::endl;
                    }
                }
                if(spikes.empty()) {
                    // nothing reads this population's spikes: the kernel still needs a queue to write
                    out << "d.spkCnt = gennmiScratch(" << batchSize << "u * (numNeurons[g] + 1u)); d.spk = d.spkCnt + " << batchSize << "u;" << std::endl;
                }
                else {
                    out << "d.numExtraSpk = " << (spikes.size() - 1) << "u;" << std::endl;
                }
                if(arch.isDelayRequired()) {
                    if(spikes.size() > 1) { unsupported("delay slots with more than one spike array on population '" + arch.getName() + "'"); }
                    out << "d.numDelaySlots = " << arch.getNumDelaySlots() << "u;" << std::endl;
                    // the reference advances spkQuePtr at the start of its neuron update (neuronUpdateGroupMerged.cc:947-953);
                    // the kernels derive the slot from the step count, the host copy is kept in step for whoever reads it
                    queue << "for(unsigned int g = 0; g < " << numGroups << "; g++)";
                    {
                        CodeStream::Scope q(queue);
                        queue << "const auto *group = &mergedNeuronUpdateGroup" << n.getIndex() << "[g];" << std::endl;
                        queue << "*" << env["_spk_que_ptr"] << " = (*" << env["_spk_que_ptr"] << " + 1) % " << arch.getNumDelaySlots() << ";" << std::endl;
                    }
                }
                // spike-like event queues ("SynSpikeEvent" children): recognised condition V > Epre of an outgoing graded projection
                const auto &events = n.getMergedSpikeEventGroups();
                for(size_t k = 0; k < events.size(); k++) {
                    auto &child = const_cast<NeuronUpdateGroupMerged::SynSpikeEvent&>(events[k]);
                    const auto &carch = child.getArchetype();
                    if(carch.getSrcNeuronGroup() != &arch || !isStaticGraded(carch.getWUInitialiser().getSnippet())) {
                        unsupported("spike-like event condition of projection '" + carch.getName() + "'");
                    }
                    const std::string sfx = "SynSpikeEvent" + std::to_string(child.getIndex());
                    EnvironmentGroupMergedField<NeuronUpdateGroupMerged::SynSpikeEvent, NeuronUpdateGroupMerged> eenv(env, child, n);
                    eenv.addField(Type::Uint32.createPointer(), "_mi_spkCntEvent", "spkCntEvent" + sfx,
                                  [&n](const auto &runtime, const auto &g, size_t i) { return runtime.getFusedEventArray(n, i, g, "SpkCntEvent"); });
                    eenv.addField(Type::Uint32.createPointer(), "_mi_spkEvent", "spkEvent" + sfx,
                                  [&n](const auto &runtime, const auto &g, size_t i) { return runtime.getFusedEventArray(n, i, g, "SpkEvent"); });
                    std::vector<Type::NumericValue> thresholds;
                    for(const auto &g : child.getGroups()) { thresholds.push_back(g.get().getWUInitialiser().getParams().at("Epre")); }
                    eenv.getStream() << "{ static const float v[] = " << table(thresholds, scalar) << "; d.spkEvent[" << k << "].spkCntEvent = gennmiDev("
                                     << eenv["_mi_spkCntEvent"] << "); d.spkEvent[" << k << "].spkEvent = gennmiDev(" << eenv["_mi_spkEvent"]
                                     << "); d.spkEvent[" << k << "].threshold = v[g]; }" << std::endl;
                    if(arch.isSpikeEventRecordingEnabled()) {
                        eenv.addField(Type::Uint32.createPointer(), "_mi_recordSpkEvent", "recordSpkEvent" + sfx,
                                      [&n](const auto &runtime, const auto &g, size_t i) { return runtime.getFusedEventArray(n, i, g, "RecordSpkEvent"); });
                        eenv.getStream() << "d.spkEvent[" << k << "].recordSpkEvent = gennmiDev(" << eenv["_mi_recordSpkEvent"] << ");" << std::endl;
                    }
                }
                out << "d.numSpkEvent = " << events.size() << "u;" << std::endl;
                // presynaptic output of outgoing projections ("OutSynPreOutput" children, neuronUpdateGroupMerged.cc:148-165)
                const auto &reverse = n.getMergedOutSynPreOutputGroups();
                for(size_t k = 0; k < reverse.size(); k++) {
                    auto &child = const_cast<NeuronUpdateGroupMerged::OutSynPreOutput&>(reverse[k]);
                    if(child.getArchetype().getPreTargetVar() != "Isyn") { unsupported("presynaptic output into a variable other than Isyn ('" + child.getArchetype().getName() + "')"); }
                    EnvironmentGroupMergedField<NeuronUpdateGroupMerged::OutSynPreOutput, NeuronUpdateGroupMerged> renv(env, child, n);
                    renv.addField(scalar.createPointer(), "_mi_outPre", "outPreOutSyn" + std::to_string(child.getIndex()),
                                  [](const auto &runtime, const auto &g, size_t) { return runtime.getArray(g, "outPre"); });
                    renv.getStream() << "d.outPre[" << k << "] = gennmiDev(" << renv["_mi_outPre"] << ");" << std::endl;
                }
                out << "d.numPreOutput = " << reverse.size() << "u;" << std::endl;
                if(arch.isSpikeTimeRequired()) { out << "d.sT = gennmiDev(" << env["_st"] << ");" << std::endl; }
                if(arch.isSpikeRecordingEnabled()) { out << "d.recordSpk = gennmiDev(" << env["_record_spk"] << ");" << std::endl; }
                out << "GENNMI_CHECK(gennmi_push_neuron_update_group(gennmiRunner, &d, nullptr));" << std::endl;
            });
    }
    body << std::endl;

    body << "void updateNeurons(" << model.getTimePrecision().getName() << " t";
    if(model.isRecordingInUse()) {
        body << ", unsigned int recordingTimestep";
    }
    body << ")";
    {
        CodeStream::Scope b(body);
        body << "gennmiEnsureFinalised();" << std::endl;
        body << queueStream.str();
        body << "GENNMI_CHECK(gennmi_step(gennmiRunner, t, " << (model.isRecordingInUse() ? "recordingTimestep" : "0u") << "));" << std::endl;
    }

    modelMerged.genMergedNeuronUpdateGroupStructs(os, *this);
    modelMerged.genMergedNeuronUpdateGroupHostStructArrayPush(os, *this);
    preambleHandler(os);
    os << bodyStream.str();
}
//--------------------------------------------------------------------------
// updateSynapses: descriptors for presynaptic and postsynaptic update groups.  The call itself only notes that
// the synaptic half of the step is due; gennmi_step() runs both halves from updateNeurons() (stepTime() always
// calls the two back to back, generateRunner.cc:270-299), which lets delay networks use a single launch.
//--------------------------------------------------------------------------
void Backend::genSynapseUpdate(CodeStream &os, FileStreamCreator, ModelSpecMerged &modelMerged,
                               BackendBase::MemorySpaces &memorySpaces, HostHandler preambleHandler) const
{
    if(m_GeneratedKernels) {
        genSynapseUpdateGenerated(os, modelMerged, memorySpaces, preambleHandler);
        return;
    }
    const ModelSpecInternal &model = modelMerged.getModel();
    const unsigned int batchSize = model.getBatchSize();
    const auto scalar = model.getPrecision();

    std::ostringstream bodyStream;
    CodeStream body(bodyStream);
    EnvironmentLibrary libEnv(body, StandardLibrary::getMathsFunctions());

    body << "void gennmiBuildSynapseGroups()";
    {
        CodeStream::Scope b(body);
        EnvironmentExternal funcEnv(libEnv);

        modelMerged.genMergedSynapseDynamicsGroups(
            *this, memorySpaces,
            [](auto &s) { unsupported("synapse dynamics code of projection '" + s.getArchetype().getName() + "'"); });

        modelMerged.genMergedPresynapticUpdateGroups(
            *this, memorySpaces,
            [this, &funcEnv, &model, batchSize, scalar](auto &s)
            {
                const auto &arch = s.getArchetype();
                const auto *wum = arch.getWUInitialiser().getSnippet();
                const unsigned int wumKind = recogniseWUM(wum, arch.getName());
                // weight-update parameters become descriptor constants too: dynamic ones are refused (see the neuron groups)
                for(const auto &g : s.getGroups()) {
                    for(const auto &p : wum->getParams()) {
                        if(g.get().isWUParamDynamic(p.name)) { unsupported("dynamic weight-update parameter '" + p.name + "' of projection '" + g.get().getName() + "'"); }
                    }
                }
                const bool srcDelay = arch.getSrcNeuronGroup()->isDelayRequired();
                const bool plastic = (wumKind == GENNMI_WUM_STDP_TRACE || wumKind == GENNMI_WUM_STDP);
                if(arch.getBackPropDelaySteps() != 0 || (plastic && (srcDelay || arch.getTrgNeuronGroup()->isDelayRequired()))) {
                    unsupported("back-propagation delay, or delay slots on a plastic projection ('" + arch.getName() + "')");
                }
                const bool graded = (wumKind == GENNMI_WUM_STATIC_GRADED);
                if((arch.isPreSpikeEventRequired() && !graded) || arch.isPostSpikeEventRequired()) { unsupported("spike-like events on projection '" + arch.getName() + "'"); }
                if(graded && srcDelay) { unsupported("delay slots on the source of graded projection '" + arch.getName() + "'"); }
                // (plastic weights, traces and spike times with a batch size above 1: one copy per batch, batch-major, which is
                // how the Runtime lays out variables with the batch dimension and how the device library indexes them)
                if(plastic && batchSize != 1 && getPreferences<Preferences>().orderedAccumulation) { unsupported("ordered accumulation of plastic weights with a batch size above 1"); }

                const auto matrixType = arch.getMatrixType();
                const bool sparse = (matrixType & SynapseMatrixConnectivity::SPARSE) && (matrixType & SynapseMatrixWeight::INDIVIDUAL);
                const bool toeplitz = (matrixType & SynapseMatrixConnectivity::TOEPLITZ) && (matrixType & SynapseMatrixWeight::KERNEL);
                const bool dense = (matrixType & SynapseMatrixConnectivity::DENSE) && (matrixType & SynapseMatrixWeight::INDIVIDUAL);
                const bool bitmask = (matrixType & SynapseMatrixConnectivity::BITMASK) != 0;
                const bool constantWeight = (wumKind == GENNMI_WUM_STATIC_PULSE_CONSTANT_WEIGHT);
                // PROCEDURAL: connectivity and weights are regenerated per spike.  The snippets arrive as code for a backend
                // to transpile; here they are recognised by identity with the built-in ones the device library implements.
                const bool procedural = (matrixType & SynapseMatrixConnectivity::PROCEDURAL) && ((matrixType & SynapseMatrixWeight::PROCEDURAL) || constantWeight);
                unsigned int procConnect = 0, procWeight = GENNMI_INIT_CONSTANT;
                std::vector<std::string> procWeightParams;
                if(procedural) {
                    const auto *conn = arch.getSparseConnectivityInitialiser().getSnippet();
                    if(conn == InitSparseConnectivitySnippet::FixedProbability::getInstance()) { procConnect = GENNMI_CONNECT_FIXED_PROBABILITY; }
                    else if(conn == InitSparseConnectivitySnippet::FixedProbabilityNoAutapse::getInstance()) { procConnect = GENNMI_CONNECT_FIXED_PROBABILITY_NO_AUTAPSE; }
                    else if(conn == InitSparseConnectivitySnippet::FixedNumberPostWithReplacement::getInstance()) { procConnect = GENNMI_CONNECT_FIXED_NUMBER_POST; }
                    else { unsupported("connectivity snippet of PROCEDURAL projection '" + arch.getName() + "' (FixedProbability, FixedProbabilityNoAutapse, FixedNumberPostWithReplacement)"); }
                    if(wumKind != GENNMI_WUM_STATIC_PULSE && !constantWeight) { unsupported("weight update model of PROCEDURAL projection '" + arch.getName() + "'"); }
                    if(!constantWeight) {
                        const auto *init = arch.getWUInitialiser().getVarInitialisers().at("g").getSnippet();
                        if(init == InitVarSnippet::Constant::getInstance()) { procWeight = GENNMI_INIT_CONSTANT; procWeightParams = {"constant"}; }
                        else if(init == InitVarSnippet::Uniform::getInstance()) { procWeight = GENNMI_INIT_UNIFORM; procWeightParams = {"min", "max"}; }
                        else if(init == InitVarSnippet::Normal::getInstance()) { procWeight = GENNMI_INIT_NORMAL; procWeightParams = {"mean", "sd"}; }
                        else if(init == InitVarSnippet::NormalClipped::getInstance()) { procWeight = GENNMI_INIT_NORMAL_CLIPPED; procWeightParams = {"mean", "sd", "min", "max"}; }
                        else if(init == InitVarSnippet::Exponential::getInstance()) { procWeight = GENNMI_INIT_EXPONENTIAL; procWeightParams = {"lambda"}; }
                        else { unsupported("weight initialisation snippet of PROCEDURAL projection '" + arch.getName() + "' (Constant, Uniform, Normal, NormalClipped, Exponential)"); }
                    }
                    if(srcDelay || arch.isDendriticOutputDelayRequired()) { unsupported("delays on PROCEDURAL projection '" + arch.getName() + "'"); }
                }
                if(!sparse && !toeplitz && !dense && !bitmask && !procedural) {
                    unsupported("matrix type of projection '" + arch.getName() + "' (SPARSE, DENSE, BITMASK, PROCEDURAL or TOEPLITZ with kernel weights)");
                }
                if(graded && !sparse) { unsupported("graded synapses on a non-SPARSE projection ('" + arch.getName() + "')"); }
                if(dense && wumKind != GENNMI_WUM_STATIC_PULSE && !constantWeight) { unsupported("weight update model of DENSE projection '" + arch.getName() + "'"); }
                if(bitmask && !constantWeight) { unsupported("weight update model of BITMASK projection '" + arch.getName() + "' (StaticPulseConstantWeight)"); }
                if(toeplitz && constantWeight) { unsupported("constant weight on Toeplitz projection '" + arch.getName() + "'"); }
                if(sparse && arch.getSparseIndType() != Type::Uint32) { unsupported("narrow sparse index type of projection '" + arch.getName() + "'"); }
                if(toeplitz) {
                    const auto *conn = arch.getToeplitzConnectivityInitialiser().getSnippet();
                    if(conn != InitToeplitzConnectivitySnippet::Conv2D::getInstance() || wumKind != GENNMI_WUM_STATIC_PULSE) {
                        unsupported("Toeplitz connectivity of projection '" + arch.getName() + "' (Conv2D with StaticPulse)");
                    }
                }

                CodeStream::Scope b(funcEnv.getStream());
                funcEnv.getStream() << "// merged presynaptic update group " << s.getIndex() << std::endl;
                funcEnv.getStream() << "for(unsigned int g = 0; g < " << s.getGroups().size() << "; g++)";
                CodeStream::Scope b2(funcEnv.getStream());
                funcEnv.getStream() << "const auto *group = &mergedPresynapticUpdateGroup" << s.getIndex() << "[g];" << std::endl;
                EnvironmentGroupMergedField<PresynapticUpdateGroupMerged> env(funcEnv, s);
                buildStandardEnvironment(env, batchSize);
                CodeStream &out = env.getStream();

                auto values = [&s](auto fn)
                {
                    std::vector<Type::NumericValue> v;
                    for(const auto &g : s.getGroups()) { v.push_back(fn(g.get())); }
                    return v;
                };
                auto counts = [&s](auto fn)
                {
                    std::vector<uint64_t> v;
                    for(const auto &g : s.getGroups()) { v.push_back(fn(g.get())); }
                    return v;
                };
                auto wuVar = [&env](const std::string &name, const Type::ResolvedType &type)
                {
                    env.addField(type.createPointer(), "_mi_" + name, name,
                                 [name](const auto &runtime, const auto &g, size_t) { return runtime.getArray(g, name); });
                    return "gennmiDev(" + env["_mi_" + name] + ")";
                };

                out << "gennmi_presynaptic_update_group_t d = {};" << std::endl;
                out << "d.matrix = " << (procedural ? GENNMI_MATRIX_PROCEDURAL : sparse ? GENNMI_MATRIX_SPARSE : (dense ? GENNMI_MATRIX_DENSE : (bitmask ? GENNMI_MATRIX_BITMASK : GENNMI_MATRIX_TOEPLITZ_CONV2D)))
                    << "u; d.wum = " << ((sparse && constantWeight) ? (unsigned int)GENNMI_WUM_STATIC_PULSE : wumKind) << "u;" << std::endl;
                if(arch.getParallelismHint() == SynapseGroup::ParallelismHint::PRESYNAPTIC) {
                    out << "d.span = " << GENNMI_SPAN_PRE << "u; d.numThreadsPerSpike = " << arch.getNumThreadsPerSpike() << "u;" << std::endl;
                }
                else {
                    out << "d.span = " << GENNMI_SPAN_AUTO << "u;" << std::endl;
                }
                out << "{ static const uint32_t a[] = " << tableU32(counts([](const SynapseGroupInternal &g){ return g.getSrcNeuronGroup()->getNumNeurons(); }))
                    << ", b[] = " << tableU32(counts([](const SynapseGroupInternal &g){ return g.getTrgNeuronGroup()->getNumNeurons(); }))
                    << ", c[] = " << tableU32(counts([this](const SynapseGroupInternal &g){ return getSynapticMatrixRowStride(g); }))
                    << "; d.numSrcNeurons = a[g]; d.numTrgNeurons = b[g]; d.rowStride = c[g]; }" << std::endl;
                if(graded) {
                    // driven by the source's event queue; V_pre is the source population's V
                    out << "d.srcSpkCnt = gennmiDev(" << env["_src_spk_cnt_event"] << "); d.srcSpk = gennmiDev(" << env["_src_spk_event"] << ");" << std::endl;
                    env.addField(scalar.createPointer(), "_mi_srcV", "V",
                                 [](const auto &runtime, const auto &g, size_t) { return g.getWUMPreNeuronVarReferences().at("V").getTargetArray(runtime); });
                    out << "d.srcV = gennmiDev(" << env["_mi_srcV"] << ");" << std::endl;
                    out << "{ static const float a[] = " << table(values([](const SynapseGroupInternal &g){ return g.getWUInitialiser().getParams().at("Epre"); }), scalar)
                        << ", b[] = " << table(values([](const SynapseGroupInternal &g){ return g.getWUInitialiser().getParams().at("Vslope"); }), scalar)
                        << "; d.gradedEpre = a[g]; d.gradedVslope = b[g]; }" << std::endl;
                }
                else {
                    out << "d.srcSpkCnt = gennmiDev(" << env["_src_spk_cnt"] << "); d.srcSpk = gennmiDev(" << env["_src_spk"] << ");" << std::endl;
                }
                if(srcDelay) {
                    if(dense || bitmask) { unsupported("axonal delay on DENSE or BITMASK projection '" + arch.getName() + "'"); }
                    out << "{ static const uint32_t a[] = " << tableU32(counts([](const SynapseGroupInternal &g){ return g.getAxonalDelaySteps(); }))
                        << ", b[] = " << tableU32(counts([](const SynapseGroupInternal &g){ return g.getSrcNeuronGroup()->getNumDelaySlots(); }))
                        << "; d.axonalDelaySteps = a[g]; d.numSrcDelaySlots = b[g]; }" << std::endl;
                }
                out << "d.outPost = gennmiDev(" << env["_out_post"] << ");" << std::endl;
                if(wumKind == GENNMI_WUM_STATIC_PULSE_REVERSE) {
                    if(!sparse || srcDelay) { unsupported("presynaptic output on a non-SPARSE or axonally delayed projection ('" + arch.getName() + "')"); }
                    out << "d.outPre = gennmiDev(" << env["_out_pre"] << ");" << std::endl;
                }
                if(constantWeight) {
                    out << "{ static const float v[] = " << table(values([](const SynapseGroupInternal &g){ return g.getWUInitialiser().getParams().at("g"); }), scalar)
                        << "; d.constantWeight = v[g]; }" << std::endl;
                    if(sparse) {
                        // the sparse kernels read a weight per synapse: the one weight is written out once, on the device
                        out << "{ const size_t count = (size_t)d.numSrcNeurons * d.rowStride; float *w = reinterpret_cast<float*>(gennmiScratch(count));" << std::endl;
                        out << "  GENNMI_CHECK(gennmi_fill_f32(w, d.constantWeight, count)); d.g = w; }" << std::endl;
                    }
                }
                else if(!procedural) {
                    out << "d.g = " << wuVar("g", scalar) << ";" << std::endl;
                }
                if(procedural) {
                    // one generator stream for the connectivity and one for the weights of every projection, numbered by
                    // the projection's place in the model's (name-ordered) list, so that a model always regenerates the same
                    // matrix: streams 2k + 1 and 2k + 2 of the model's seed
                    auto place = [&model](const SynapseGroupInternal &g) -> uint64_t
                    {
                        return (uint64_t)std::distance(model.getSynapseGroups().cbegin(), model.getSynapseGroups().find(g.getName()));
                    };
                    out << "d.procedural.seed = " << model.getSeed() << "ull; d.procedural.connectivity = " << procConnect << "u; d.procedural.weightSnippet = "
                        << procWeight << "u;" << std::endl;
                    out << "{ static const uint32_t a[] = " << tableU32(counts([&place](const SynapseGroupInternal &g){ return 2 * place(g) + 1; }))
                        << ", b[] = " << tableU32(counts([&place](const SynapseGroupInternal &g){ return 2 * place(g) + 2; }))
                        << "; d.procedural.connectivityStream = a[g]; d.procedural.weightStream = b[g]; }" << std::endl;
                    if(procConnect == GENNMI_CONNECT_FIXED_NUMBER_POST) {
                        out << "{ static const uint32_t v[] = " << tableU32(counts([](const SynapseGroupInternal &g)
                            { return (uint64_t)g.getSparseConnectivityInitialiser().getParams().at("num").template cast<unsigned int>(); }))
                            << "; d.procedural.num = v[g]; }" << std::endl;
                    }
                    else {
                        out << "{ static const double v[] = " << table(values([](const SynapseGroupInternal &g)
                            { return g.getSparseConnectivityInitialiser().getParams().at("prob"); }), Type::Double) << "; d.procedural.prob = v[g]; }" << std::endl;
                    }
                    for(size_t k = 0; k < procWeightParams.size(); k++) {
                        const std::string name = procWeightParams[k];
                        out << "{ static const double v[] = " << table(values([name](const SynapseGroupInternal &g)
                            { return g.getWUInitialiser().getVarInitialisers().at("g").getParams().at(name); }), Type::Double)
                            << "; d.procedural.weightParams[" << k << "] = v[g]; }" << std::endl;
                    }
                }
                if(sparse) {
                    out << "d.rowLength = gennmiDev(" << env["_row_length"] << "); d.ind = gennmiDev(" << env["_ind"] << ");" << std::endl;
                }
                else if(bitmask) {
                    out << "d.gp = gennmiDev(" << env["_gp"] << ");" << std::endl;
                }
                else if(toeplitz) {
                    const auto &names = std::vector<std::string>{"conv_kh", "conv_kw", "conv_ih", "conv_iw", "conv_ic", "conv_oh", "conv_ow", "conv_oc"};
                    for(size_t k = 0; k < names.size(); k++) {
                        out << "{ static const int32_t v[] = " << tableU32(counts([&names, k](const SynapseGroupInternal &g)
                            { return (uint64_t)g.getToeplitzConnectivityInitialiser().getParams().at(names[k]).template cast<int>(); }))
                            << "; d.conv[" << k << "] = v[g]; }" << std::endl;
                    }
                }
                if(wumKind == GENNMI_WUM_STATIC_PULSE_DENDRITIC_DELAY) {
                    out << "d.d = " << wuVar("d", Type::Uint8) << "; d.denDelay = gennmiDev(" << env["_den_delay"] << "); d.denDelayPtr = gennmiDev(" << env["_den_delay_ptr"] << ");" << std::endl;
                    out << "{ static const uint32_t v[] = " << tableU32(counts([](const SynapseGroupInternal &g){ return g.getMaxDendriticDelayTimesteps(); })) << "; d.maxDenDelay = v[g]; }" << std::endl;
                }
                if(wumKind == GENNMI_WUM_STDP) {
                    out << "d.trgST = gennmiDev(" << env["_trg_st"] << ");" << std::endl;
                    for(const auto &[field, p] : {std::pair<const char*, const char*>{"tauMinus", "tauMinus"}, {"aMinus", "Aminus"}, {"wMin", "Wmin"}, {"wMax", "Wmax"}}) {
                        const std::string param = p;
                        out << "{ static const float v[] = " << table(values([param](const SynapseGroupInternal &g){ return g.getWUInitialiser().getParams().at(param); }), scalar)
                            << "; d." << field << " = v[g]; }" << std::endl;
                    }
                }
                if(wumKind == GENNMI_WUM_STDP_TRACE) {
                    env.addField(scalar.createPointer(), "_mi_postTrace", "postTrace",
                                 [](const auto &runtime, const auto &g, size_t) { return runtime.getArray(g.getFusedWUPostTarget(), "postTrace"); });
                    out << "d.trgST = gennmiDev(" << env["_trg_st"] << "); d.postTrace = gennmiDev(" << env["_mi_postTrace"] << ");" << std::endl;
                    for(const char *p : {"aMinus", "wMin", "wMax"}) {
                        out << "{ static const float v[] = " << table(values([p](const SynapseGroupInternal &g){ return g.getWUInitialiser().getParams().at(p); }), scalar)
                            << "; d." << p << " = v[g]; }" << std::endl;
                    }
                }
                out << "GENNMI_CHECK(gennmi_push_presynaptic_update_group(gennmiRunner, &d, nullptr));" << std::endl;
            });

        modelMerged.genMergedPostsynapticUpdateGroups(
            *this, memorySpaces,
            [this, &funcEnv, batchSize, scalar](auto &s)
            {
                const auto &arch = s.getArchetype();
                const bool additive = isAdditiveSTDP(arch.getWUInitialiser().getSnippet());
                if(!additive && !isTraceSTDP(arch.getWUInitialiser().getSnippet())) { unsupported("postsynaptic-spike code of projection '" + arch.getName() + "'"); }
                if(!(arch.getMatrixType() & SynapseMatrixConnectivity::SPARSE)) { unsupported("postsynaptic learning on a non-SPARSE projection"); }

                CodeStream::Scope b(funcEnv.getStream());
                funcEnv.getStream() << "// merged postsynaptic update group " << s.getIndex() << std::endl;
                funcEnv.getStream() << "for(unsigned int g = 0; g < " << s.getGroups().size() << "; g++)";
                CodeStream::Scope b2(funcEnv.getStream());
                funcEnv.getStream() << "const auto *group = &mergedPostsynapticUpdateGroup" << s.getIndex() << "[g];" << std::endl;
                EnvironmentGroupMergedField<PostsynapticUpdateGroupMerged> env(funcEnv, s);
                buildStandardEnvironment(env, batchSize);
                CodeStream &out = env.getStream();
                auto counts = [&s](auto fn)
                {
                    std::vector<uint64_t> v;
                    for(const auto &g : s.getGroups()) { v.push_back(fn(g.get())); }
                    return v;
                };
                env.addField(scalar.createPointer(), "_mi_g", "g", [](const auto &runtime, const auto &g, size_t) { return runtime.getArray(g, "g"); });
                if(!additive) {
                    env.addField(scalar.createPointer(), "_mi_preTrace", "preTrace",
                                 [](const auto &runtime, const auto &g, size_t) { return runtime.getArray(g.getFusedWUPreTarget(), "preTrace"); });
                }
                out << "gennmi_postsynaptic_update_group_t d = {};" << std::endl;
                out << "{ static const uint32_t a[] = " << tableU32(counts([](const SynapseGroupInternal &g){ return g.getSrcNeuronGroup()->getNumNeurons(); }))
                    << ", b[] = " << tableU32(counts([](const SynapseGroupInternal &g){ return g.getTrgNeuronGroup()->getNumNeurons(); }))
                    << ", c[] = " << tableU32(counts([this](const SynapseGroupInternal &g){ return getSynapticMatrixRowStride(g); }))
                    << ", e[] = " << tableU32(counts([](const SynapseGroupInternal &g){ return g.getMaxSourceConnections(); }))
                    << "; d.numSrcNeurons = a[g]; d.numTrgNeurons = b[g]; d.rowStride = c[g]; d.colStride = e[g]; }" << std::endl;
                out << "d.colLength = gennmiDev(" << env["_col_length"] << "); d.remap = gennmiDev(" << env["_remap"] << "); d.g = gennmiDev(" << env["_mi_g"] << ");" << std::endl;
                out << "d.trgSpkCnt = gennmiDev(" << env["_trg_spk_cnt"] << "); d.trgSpk = gennmiDev(" << env["_trg_spk"] << ");" << std::endl;
                out << "d.srcST = gennmiDev(" << env["_src_st"] << ");" << std::endl;
                if(!additive) { out << "d.preTrace = gennmiDev(" << env["_mi_preTrace"] << ");" << std::endl; }
                out << "d.rowLength = gennmiDev(" << env["_row_length"] << "); d.ind = gennmiDev(" << env["_ind"] << ");" << std::endl;
                const std::vector<std::pair<std::string, std::string>> fields = additive
                    ? std::vector<std::pair<std::string, std::string>>{{"tauPlus", "tauPlus"}, {"aPlus", "Aplus"}, {"wMin", "Wmin"}, {"wMax", "Wmax"}}
                    : std::vector<std::pair<std::string, std::string>>{{"aPlus", "aPlus"}, {"wMin", "wMin"}, {"wMax", "wMax"}};
                for(const auto &[field, p] : fields) {
                    std::vector<Type::NumericValue> v;
                    for(const auto &g : s.getGroups()) { v.push_back(g.get().getWUInitialiser().getParams().at(p)); }
                    out << "{ static const float v[] = " << table(v, scalar) << "; d." << field << " = v[g]; }" << std::endl;
                }
                out << "GENNMI_CHECK(gennmi_push_postsynaptic_update_group(gennmiRunner, &d, nullptr));" << std::endl;
            });
    }
    body << std::endl;
    body << "void updateSynapses(" << model.getTimePrecision().getName() << ")";
    {
        CodeStream::Scope b(body);
        body << "// runs as part of updateNeurons()" << std::endl;
    }

    modelMerged.genMergedPresynapticUpdateGroupStructs(os, *this);
    modelMerged.genMergedPostsynapticUpdateGroupStructs(os, *this);
    modelMerged.genMergedPresynapticUpdateGroupHostStructArrayPush(os, *this);
    modelMerged.genMergedPostsynapticUpdateGroupHostStructArrayPush(os, *this);
    preambleHandler(os);
    os << bodyStream.str();
}
//--------------------------------------------------------------------------
void Backend::genCustomUpdate(CodeStream &os, FileStreamCreator, ModelSpecMerged &modelMerged,
                              BackendBase::MemorySpaces &memorySpaces, HostHandler preambleHandler) const
{
    // custom update code is arbitrary model code: its kernels are generated, whichever kernels the step runs on
    // (Optimiser::createBackend tells the backend that the model has any)
    if(hasDeviceModules()) {
        if(!m_GeneratedKernels && !modelMerged.getModel().getCustomConnectivityUpdates().empty()) {
            unsupported("custom connectivity updates beside the device library's step kernels, whose launch plans rely on rows sorted by target (Preferences::kernelSource AUTO or GENERATED generates the step's kernels)");
        }
        genCustomUpdateGenerated(os, modelMerged, memorySpaces, preambleHandler);
        return;
    }
    const ModelSpecInternal &model = modelMerged.getModel();
    if(!model.getCustomUpdates().empty() || !model.getCustomWUUpdates().empty() || !model.getCustomConnectivityUpdates().empty()) {
        unsupported("custom updates with a backend object that was not told of them (create it with Optimiser::createBackend)");
    }
    preambleHandler(os);
}
//--------------------------------------------------------------------------
// initialize() / initializeSparse(): the reference's generic initialisation code, generated as plain host loops over
// the arrays' host buffers (merged init groups carry host pointers), followed by an upload of every buffer.
// initializeSparse() additionally builds the column view of plastic projections on the device.
//--------------------------------------------------------------------------
namespace
{
// value snippets the device library draws itself: snippet id and parameter names in the order gennmi_init_var takes them
bool deviceVarSnippet(const InitVarSnippet::Base *snippet, unsigned int &id, std::vector<std::string> &params)
{
    if(snippet == InitVarSnippet::Constant::getInstance()) { id = GENNMI_INIT_CONSTANT; params = {"constant"}; }
    else if(snippet == InitVarSnippet::Uniform::getInstance()) { id = GENNMI_INIT_UNIFORM; params = {"min", "max"}; }
    else if(snippet == InitVarSnippet::Normal::getInstance()) { id = GENNMI_INIT_NORMAL; params = {"mean", "sd"}; }
    else if(snippet == InitVarSnippet::NormalClipped::getInstance()) { id = GENNMI_INIT_NORMAL_CLIPPED; params = {"mean", "sd", "min", "max"}; }
    else if(snippet == InitVarSnippet::Exponential::getInstance()) { id = GENNMI_INIT_EXPONENTIAL; params = {"lambda"}; }
    else if(snippet == InitVarSnippet::Gamma::getInstance()) { id = GENNMI_INIT_GAMMA; params = {"a", "b"}; }
    else { return false; }
    return true;
}
}

void Backend::genInit(CodeStream &os, FileStreamCreator, ModelSpecMerged &modelMerged,
                      BackendBase::MemorySpaces &memorySpaces, HostHandler preambleHandler) const
{
    const ModelSpecInternal &model = modelMerged.getModel();
    const unsigned int batchSize = model.getBatchSize();
    const bool deviceInit = getPreferences<Preferences>().deviceInitialisation;
    // generator streams of device-side initialisation: 2k + 1 for the connectivity of the k-th projection by name (the numbering
    // PROCEDURAL projections use for the same purpose), 2k + 2 + 2 * (number of projections) * v for its v-th variable by name
    auto place = [&model](const SynapseGroupInternal &g) -> uint64_t
    {
        return (uint64_t)std::distance(model.getSynapseGroups().cbegin(), model.getSynapseGroups().find(g.getName()));
    };
    const uint64_t numProjections = model.getSynapseGroups().size();
    // Generator streams are numbered in ranges per consumer under one key (the model's seed): initialisation arrays from 1
    // (2k + 1, 2k + 2 + 2 P v), current sources from 1000, neuron code from 2000, weight-update code from 3000 (eight per
    // projection), custom connectivity updates from 6000, neuron variable initialisation from 8000 (sixteen per population).
    // A model large enough for two ranges to meet would draw the same
    // words in two places, so it is refused here rather than simulated with correlated noise.
    {
        size_t maxVars = 0;
        for(const auto &g : model.getSynapseGroups()) { maxVars = std::max(maxVars, g.second.getWUInitialiser().getSnippet()->getVars().size()); }
        size_t numCurrentSources = 0;
        for(const auto &n : model.getNeuronGroups()) { numCurrentSources += n.second.getCurrentSources().size(); }
        if(2 * numProjections * (maxVars + 1) + 2 >= 1000 || numCurrentSources >= 1000 || model.getNeuronGroups().size() >= 1000 || numProjections >= 375) {
            unsupported("a model of this many groups (the counter-based generator's stream ranges of initialisation arrays, current sources, "
                        "neuron code and weight-update code would overlap)");
        }
    }
    // the model's seed, or one drawn when the runner is loaded (ModelSpec: seed 0 = a different one every run)
    const std::string seedExpr = (model.getSeed() != 0) ? (std::to_string(model.getSeed()) + "ull")
                                                        : std::string("gennmiRandomSeed()");

    // Per-synapse variables whose initialisers are all value snippets the device library draws itself
    // (Preferences::deviceInitialisation), of every projection of merged group `s`: one gennmi_init_var per variable over
    // `count` elements (padding of sparse rows included: it is never read), and a note that the device now holds the array.
    // False, and nothing emitted, when some variable needs the reference's host code.
    auto emitDeviceVars = [&](auto &s, auto &env, const std::string &count) -> bool
    {
        if(!deviceInit || !s.getArchetype().isWUVarInitRequired() || batchSize != 1) { return false; }
        struct DeviceVar { std::string name; unsigned int snippet; std::vector<std::string> params; };
        std::vector<DeviceVar> deviceVars;
        for(const auto &var : s.getArchetype().getWUInitialiser().getSnippet()->getVars()) {
            const auto &init = s.getArchetype().getWUInitialiser().getVarInitialisers().at(var.name);
            if(Utils::areTokensEmpty(init.getCodeTokens()) || init.isKernelRequired()) { continue; }    // nothing to do here
            DeviceVar d{var.name, 0, {}};
            if(var.type.resolve(model.getTypeContext()) != Type::Float || !deviceVarSnippet(init.getSnippet(), d.snippet, d.params)) { return false; }
            for(const auto &g : s.getGroups()) {
                if(g.get().getWUInitialiser().getVarInitialisers().at(var.name).getSnippet() != init.getSnippet()) { return false; }
            }
            deviceVars.push_back(d);
        }
        size_t varIndex = 0;
        for(const auto &d : deviceVars) {
            const std::string name = d.name;
            env.addField(Type::Float.createPointer(), "_mi_init_" + name, name,
                         [name](const auto &runtime, const auto &g, size_t) { return runtime.getArray(g, name); });
            std::vector<uint64_t> streams;
            for(const auto &g : s.getGroups()) { streams.push_back(2 * place(g.get()) + 2 + 2 * numProjections * varIndex); }
            CodeStream::Scope scope(env.getStream());
            env.getStream() << "static const uint32_t stream[] = " << tableU32(streams) << ";" << std::endl;
            env.getStream() << "double params[4] = {0.0, 0.0, 0.0, 0.0};" << std::endl;
            for(size_t k = 0; k < d.params.size(); k++) {
                std::vector<Type::NumericValue> values;
                for(const auto &g : s.getGroups()) { values.push_back(g.get().getWUInitialiser().getVarInitialisers().at(name).getParams().at(d.params[k])); }
                env.getStream() << "{ static const double v[] = " << table(values, Type::Double) << "; params[" << k << "] = v[g]; }" << std::endl;
            }
            env.getStream() << "GENNMI_CHECK(gennmi_init_var(gennmiDev(" << env["_mi_init_" + name] << "), " << GENNMI_TYPE_F32 << "u, " << count << ", "
                            << d.snippet << "u, params, " << seedExpr << ", stream[g]));" << std::endl;
            env.getStream() << "GENNMI_CHECK(gennmi_mirror_device_initialised(" << env["_mi_init_" + name] << "));" << std::endl;
            varIndex++;
        }
        return true;
    };

    std::ostringstream bodyStream;
    CodeStream body(bodyStream);
    EnvironmentLibrary rngEnv(body, StandardLibrary::getHostRNGFunctions(model.getPrecision()));
    EnvironmentLibrary initEnv(rngEnv, StandardLibrary::getMathsFunctions());

    // "for every group of this merged group" wrapper shared by all init groups
    auto forEachGroup = [](EnvironmentExternalBase &funcEnv, const std::string &structName, size_t index, size_t numGroups, auto emit)
    {
        CodeStream::Scope b(funcEnv.getStream());
        funcEnv.getStream() << "// merged " << structName << " " << index << std::endl;
        funcEnv.getStream() << "for(unsigned int g = 0; g < " << numGroups << "; g++)";
        CodeStream::Scope b2(funcEnv.getStream());
        funcEnv.getStream() << "const auto *group = &merged" << structName << index << "[g];" << std::endl;
        emit();
    };

    // initTime / initSparseTime (generateRunner.cc:161-162): initialisation runs on the host and ends with an upload, so the
    // counters are wall-clock time of the whole function, taken when the model enables timing as the reference's are
    const bool timing = model.isTimingEnabled();
    const std::string timerStart = "const auto gennmiInitStart = std::chrono::steady_clock::now();";
    auto timerStop = [](const std::string &counter)
    {
        return counter + " += std::chrono::duration<double>(std::chrono::steady_clock::now() - gennmiInitStart).count();";
    };
    body << "void initialize()";
    {
        CodeStream::Scope b(body);
        if(timing) { body << timerStart << std::endl; }
        body << "GENNMI_CHECK(gennmi_mirrors_begin_initialisation());" << std::endl;
        EnvironmentExternal funcEnv(initEnv);
        funcEnv.add(model.getTimePrecision().addConst(), "dt", Type::writeNumeric(model.getDT(), model.getTimePrecision()));

        modelMerged.genMergedNeuronInitGroups(
            *this, memorySpaces,
            [&](auto &n)
            {
                forEachGroup(funcEnv, "NeuronInitGroup", n.getIndex(), n.getGroups().size(), [&]
                {
                    EnvironmentGroupMergedField<NeuronInitGroupMerged> env(funcEnv, n);
                    buildStandardEnvironment(env, batchSize);
                    // neuron variables whose initialiser is a value snippet the device draws (Preferences::deviceInitialisation):
                    // one gennmi_init_var each; genVariableInit then leaves their host loops out of the generic code below.
                    // Streams 8000 + 16 * (the population's place by name) + the variable's place in the model.
                    m_DeviceInitialisedVars.clear();
                    if(deviceInit && batchSize == 1) {
                        const auto &arch = n.getArchetype();
                        const auto vars = arch.getModel()->getVars();
                        for(size_t v = 0; v < vars.size() && v < 16; v++) {
                            const auto &var = vars[v];
                            const auto &init = arch.getVarInitialisers().at(var.name);
                            unsigned int snippet = 0;
                            std::vector<std::string> paramNames;
                            bool eligible = !Utils::areTokensEmpty(init.getCodeTokens()) && var.type.resolve(model.getTypeContext()) == Type::Float
                                            && (getVarAccessDim(var.access) & VarAccessDim::ELEMENT) && !arch.isVarQueueRequired(var.name)
                                            && deviceVarSnippet(init.getSnippet(), snippet, paramNames);
                            for(const auto &g : n.getGroups()) {
                                eligible = eligible && (g.get().getVarInitialisers().at(var.name).getSnippet() == init.getSnippet()) && !g.get().isVarQueueRequired(var.name);
                            }
                            if(!eligible) { continue; }
                            const std::string name = var.name;
                            env.addField(Type::Float.createPointer(), "_mi_init_" + name, name,
                                         [name](const auto &runtime, const auto &g, size_t) { return runtime.getArray(g, name); });
                            std::vector<uint64_t> streams;
                            for(const auto &g : n.getGroups()) {
                                streams.push_back(8000 + 16 * (uint64_t)std::distance(model.getNeuronGroups().cbegin(), model.getNeuronGroups().find(g.get().getName())) + v);
                            }
                            CodeStream::Scope scope(env.getStream());
                            env.getStream() << "static const uint32_t stream[] = " << tableU32(streams) << ";" << std::endl;
                            env.getStream() << "double params[4] = {0.0, 0.0, 0.0, 0.0};" << std::endl;
                            for(size_t k = 0; k < paramNames.size(); k++) {
                                std::vector<Type::NumericValue> values;
                                for(const auto &g : n.getGroups()) { values.push_back(g.get().getVarInitialisers().at(name).getParams().at(paramNames[k])); }
                                env.getStream() << "{ static const double v[] = " << table(values, Type::Double) << "; params[" << k << "] = v[g]; }" << std::endl;
                            }
                            env.getStream() << "GENNMI_CHECK(gennmi_init_var(gennmiDev(" << env["_mi_init_" + name] << "), " << GENNMI_TYPE_F32 << "u, (size_t)" << env["num_neurons"]
                                            << ", " << snippet << "u, params, " << seedExpr << ", stream[g]));" << std::endl;
                            env.getStream() << "GENNMI_CHECK(gennmi_mirror_device_initialised(" << env["_mi_init_" + name] << "));" << std::endl;
                            m_DeviceInitialisedVars.insert(name);
                        }
                    }
                    n.generateInit(*this, env, batchSize);
                    m_DeviceInitialisedVars.clear();
                });
            });
        modelMerged.genMergedSynapseInitGroups(
            *this, memorySpaces,
            [&](auto &s)
            {
                forEachGroup(funcEnv, "SynapseInitGroup", s.getIndex(), s.getGroups().size(), [&]
                {
                    EnvironmentGroupMergedField<SynapseInitGroupMerged> env(funcEnv, s);
                    buildStandardEnvironment(env, batchSize);
                    // variables of DENSE matrices and of kernels (initGroupMerged.cc:563-593): drawn on the device where every
                    // one of them can be, else the reference's loops on the host
                    const bool kernel = (s.getArchetype().getMatrixType() & SynapseMatrixWeight::KERNEL);
                    if(!emitDeviceVars(s, env, kernel ? ("(size_t)" + env["_kernel_size"]) : ("(size_t)" + env["num_pre"] + " * " + env["_row_stride"]))) {
                        s.generateInit(*this, env, batchSize);
                    }
                });
            });
        // variables of custom updates (per neuron, and per synapse of DENSE and KERNEL matrices)
        modelMerged.genMergedCustomUpdateInitGroups(
            *this, memorySpaces,
            [&](auto &c)
            {
                forEachGroup(funcEnv, "CustomUpdateInitGroup", c.getIndex(), c.getGroups().size(), [&]
                {
                    EnvironmentGroupMergedField<CustomUpdateInitGroupMerged> env(funcEnv, c);
                    buildStandardEnvironment(env, batchSize);
                    c.generateInit(*this, env, batchSize);
                });
            });
        modelMerged.genMergedCustomWUUpdateInitGroups(
            *this, memorySpaces,
            [&](auto &c)
            {
                forEachGroup(funcEnv, "CustomWUUpdateInitGroup", c.getIndex(), c.getGroups().size(), [&]
                {
                    EnvironmentGroupMergedField<CustomWUUpdateInitGroupMerged> env(funcEnv, c);
                    buildStandardEnvironment(env, batchSize);
                    c.generateInit(*this, env, batchSize);
                });
            });
        // presynaptic and postsynaptic variables of custom connectivity updates
        modelMerged.genMergedCustomConnectivityUpdatePreInitGroups(
            *this, memorySpaces,
            [&](auto &c)
            {
                forEachGroup(funcEnv, "CustomConnectivityUpdatePreInitGroup", c.getIndex(), c.getGroups().size(), [&]
                {
                    EnvironmentGroupMergedField<CustomConnectivityUpdatePreInitGroupMerged> env(funcEnv, c);
                    buildStandardEnvironment(env);
                    c.generateInit(*this, env, batchSize);
                });
            });
        modelMerged.genMergedCustomConnectivityUpdatePostInitGroups(
            *this, memorySpaces,
            [&](auto &c)
            {
                forEachGroup(funcEnv, "CustomConnectivityUpdatePostInitGroup", c.getIndex(), c.getGroups().size(), [&]
                {
                    EnvironmentGroupMergedField<CustomConnectivityUpdatePostInitGroupMerged> env(funcEnv, c);
                    buildStandardEnvironment(env);
                    c.generateInit(*this, env, batchSize);
                });
            });
        modelMerged.genMergedSynapseConnectivityInitGroups(
            *this, memorySpaces,
            [&](auto &s)
            {
                const auto &arch = s.getArchetype();
                const auto &connect = arch.getSparseConnectivityInitialiser();
                if(!(arch.getMatrixType() & SynapseMatrixConnectivity::SPARSE)) {
                    unsupported("connectivity initialisation of projection '" + arch.getName() + "' (SPARSE only)");
                }
                const bool byRow = !Utils::areTokensEmpty(connect.getRowBuildCodeTokens());
                // built-in snippets the device library generates itself (Preferences::deviceInitialisation)
                const auto *snippet = connect.getSnippet();
                int deviceSnippet = !deviceInit ? -1
                    : (snippet == InitSparseConnectivitySnippet::FixedProbability::getInstance()) ? 0
                    : (snippet == InitSparseConnectivitySnippet::FixedProbabilityNoAutapse::getInstance()) ? 1
                    : (snippet == InitSparseConnectivitySnippet::FixedNumberPostWithReplacement::getInstance()) ? 2
                    : (snippet == InitSparseConnectivitySnippet::OneToOne::getInstance()) ? 3
                    : (snippet == InitSparseConnectivitySnippet::FixedNumberPreWithReplacement::getInstance()) ? 4
                    : (snippet == InitSparseConnectivitySnippet::Conv2D::getInstance()) ? 5 : -1;
                // per-synapse variables initialised from a kernel (the synapse's position in it is only known while its row is
                // built): on the device when each is a float copy of a kernel entry (InitVarSnippet::Kernel)
                std::vector<std::string> kernelVars;
                for(const auto &var : arch.getWUInitialiser().getSnippet()->getVars()) {
                    const auto &init = arch.getWUInitialiser().getVarInitialisers().at(var.name);
                    if(Utils::areTokensEmpty(init.getCodeTokens()) || !init.isKernelRequired()) { continue; }
                    kernelVars.push_back(var.name);
                    bool eligible = (deviceSnippet == 5) && (batchSize == 1) && var.type.resolve(model.getTypeContext()) == Type::Float;
                    for(const auto &g : s.getGroups()) {
                        eligible = eligible && (g.get().getWUInitialiser().getVarInitialisers().at(var.name).getSnippet() == InitVarSnippet::Kernel::getInstance());
                    }
                    if(!eligible) { deviceSnippet = -1; }
                }
                if(deviceSnippet != 5 && !kernelVars.empty() && deviceSnippet >= 0) { deviceSnippet = -1; }
                if(deviceSnippet >= 0) {
                    forEachGroup(funcEnv, "SynapseConnectivityInitGroup", s.getIndex(), s.getGroups().size(), [&]
                    {
                        EnvironmentGroupMergedField<SynapseConnectivityInitGroupMerged> env(funcEnv, s);
                        buildStandardEnvironment(env, batchSize);
                        std::vector<uint64_t> streams;
                        std::vector<Type::NumericValue> values;
                        for(const auto &g : s.getGroups()) {
                            streams.push_back(2 * place(g.get()) + 1);
                            const auto &params = g.get().getSparseConnectivityInitialiser().getParams();
                            if(deviceSnippet <= 1) { values.push_back(params.at("prob")); }
                            else if(deviceSnippet == 2 || deviceSnippet == 4) { values.push_back(params.at("num")); }
                            else if(deviceSnippet == 5) {
                                for(const char *name : {"conv_kh", "conv_kw", "conv_sh", "conv_sw", "conv_padh", "conv_padw", "conv_ih", "conv_iw", "conv_ic",
                                                        "conv_oh", "conv_ow", "conv_oc"}) {
                                    values.push_back(params.at(name));
                                }
                            }
                        }
                        CodeStream::Scope scope(env.getStream());
                        env.getStream() << "static const uint32_t stream[] = " << tableU32(streams) << ";" << std::endl;
                        if(deviceSnippet != 3) { env.getStream() << "static const double value[] = " << table(values, Type::Double) << ";" << std::endl; }
                        env.getStream() << "uint32_t overflowRows = 0;" << std::endl;
                        const std::string arrays = "gennmiDev(" + env["_row_length"] + "), gennmiDev(" + env["_ind"] + ")";
                        const std::string shape = env["num_pre"] + ", " + env["num_post"] + ", " + env["_row_stride"];
                        if(deviceSnippet <= 1) {
                            env.getStream() << "GENNMI_CHECK(gennmi_init_sparse_fixed_probability(" << shape << ", value[g], " << deviceSnippet << ", " << seedExpr
                                            << ", stream[g], " << arrays << ", &overflowRows));" << std::endl;
                        }
                        else if(deviceSnippet == 2) {
                            env.getStream() << "GENNMI_CHECK(gennmi_init_sparse_fixed_number_post(" << shape << ", (uint32_t)value[g], nullptr, " << seedExpr
                                            << ", stream[g], " << arrays << ", &overflowRows));" << std::endl;
                        }
                        else if(deviceSnippet == 3) {
                            env.getStream() << "(void)stream; GENNMI_CHECK(gennmi_init_sparse_one_to_one(" << shape << ", " << arrays << "));" << std::endl;
                        }
                        else if(deviceSnippet == 4) {
                            env.getStream() << "GENNMI_CHECK(gennmi_init_sparse_fixed_number_pre(" << shape << ", (uint32_t)value[g], " << seedExpr
                                            << ", stream[g], " << arrays << ", &overflowRows));" << std::endl;
                        }
                        else {
                            env.getStream() << "(void)stream; int32_t conv[12]; for(int k = 0; k < 12; k++) { conv[k] = (int32_t)value[12 * g + k]; }" << std::endl;
                            env.getStream() << "if((unsigned long long)conv[6] * conv[7] * conv[8] != " << env["num_pre"] << " || (unsigned long long)conv[9] * conv[10] * conv[11] != "
                                            << env["num_post"] << ") { throw std::runtime_error(\"Conv2D connectivity: shapes do not match the populations' sizes\"); }" << std::endl;
                            env.getStream() << "GENNMI_CHECK(gennmi_init_sparse_conv2d(conv, " << env["_row_stride"] << ", " << arrays << ", nullptr, nullptr, &overflowRows));" << std::endl;
                            // weights that are kernel entries are written beside the connectivity (the row build is repeated per variable)
                            for(const auto &name : kernelVars) {
                                EnvironmentGroupMergedField<SynapseConnectivityInitGroupMerged> varEnv(env, s);
                                varEnv.addExtraGlobalParams(InitVarSnippet::Kernel::getInstance()->getExtraGlobalParams(), name);
                                varEnv.addField(Type::Float.createPointer(), "_mi_kernel_var", name,
                                                [name](const auto &runtime, const auto &g, size_t) { return runtime.getArray(g, name); });
                                varEnv.getStream() << "GENNMI_CHECK(gennmi_init_sparse_conv2d(conv, " << env["_row_stride"] << ", " << arrays << ", gennmiDev(" << varEnv["kernel"]
                                                   << "), gennmiDev(" << varEnv["_mi_kernel_var"] << "), &overflowRows));" << std::endl;
                                varEnv.getStream() << "GENNMI_CHECK(gennmi_mirror_device_initialised(" << varEnv["_mi_kernel_var"] << "));" << std::endl;
                            }
                        }
                        // the device holds the matrix: the upload that ends initialize() leaves it alone, and host code that reads
                        // rows (per-row initialisation code) asks for the copy first
                        env.getStream() << "GENNMI_CHECK(gennmi_mirror_device_initialised(" << env["_row_length"] << "));" << std::endl;
                        env.getStream() << "GENNMI_CHECK(gennmi_mirror_device_initialised(" << env["_ind"] << "));" << std::endl;
                    });
                    return;
                }
                forEachGroup(funcEnv, "SynapseConnectivityInitGroup", s.getIndex(), s.getGroups().size(), [&]
                {
                    EnvironmentGroupMergedField<SynapseConnectivityInitGroupMerged> env(funcEnv, s);
                    buildStandardEnvironment(env, batchSize);
                    // rows start empty whatever an earlier initialize() left behind
                    env.printLine("std::fill_n($(_row_length), $(num_pre), 0u);");
                    if(byRow) {
                        env.print("for(unsigned int i = 0; i < $(num_pre); i++)");
                        env.add(Type::Uint32.addConst(), "id_pre", "i");
                        env.add(Type::Uint32.addConst(), "id_post_begin", "0");
                    }
                    else {
                        env.print("for(unsigned int j = 0; j < $(num_post); j++)");
                        env.add(Type::Uint32.addConst(), "id_post", "j");
                        env.add(Type::Uint32.addConst(), "id_pre_begin", "0");
                    }
                    env.add(Type::Uint32.addConst(), "id_thread", "0");
                    env.add(Type::Uint32.addConst(), "num_threads", "1");
                    CodeStream::Scope loop(env.getStream());

                    // addSynapse(other end of the synapse): append to the row
                    std::ostringstream addStream;
                    CodeStream add(addStream);
                    {
                        CodeStream::Scope a(add);
                        EnvironmentExternal addEnv(env, add);
                        if(byRow) {
                            addEnv.add(Type::Uint32.addConst(), "id_post", "idPost", {addEnv.addInitialiser("const unsigned int idPost = $(0);")});
                        }
                        else {
                            addEnv.add(Type::Uint32.addConst(), "id_pre", "idPre", {addEnv.addInitialiser("const unsigned int idPre = $(0);")});
                        }
                        addEnv.add(Type::Uint32.addConst(), "id_syn", "idSyn",
                                   {addEnv.addInitialiser("const unsigned int idSyn = ($(id_pre) * $(_row_stride)) + $(_row_length)[$(id_pre)];")});
                        if(!arch.getKernelSize().empty()) {
                            // variables that are functions of the synapse's position in the kernel: addSynapse's further arguments
                            // name it (single_threaded_cpu/backend.cc:1200-1215)
                            EnvironmentGroupMergedField<SynapseConnectivityInitGroupMerged> kernelEnv(addEnv, s);
                            for(size_t k = 0; k < arch.getKernelSize().size(); k++) {
                                const std::string index = std::to_string(k);
                                kernelEnv.add(Type::Uint32.addConst(), "id_kernel_" + index, "idKernel" + index,
                                              {kernelEnv.addInitialiser("const unsigned int idKernel" + index + " = $(" + std::to_string(k + 1) + ");")});
                            }
                            s.generateKernelInit(kernelEnv, batchSize);
                        }
                        addEnv.printLine("$(_ind)[$(id_syn)] = $(id_post);");
                        addEnv.printLine("$(_row_length)[$(id_pre)]++;");
                    }
                    env.add(Type::ResolvedType::createFunction(Type::Void, std::vector<Type::ResolvedType>(1 + arch.getKernelSize().size(), Type::Uint32)),
                            "addSynapse", addStream.str());
                    if(byRow) {
                        s.generateSparseRowInit(env);
                    }
                    else {
                        s.generateSparseColumnInit(env);
                    }
                });
            });
        funcEnv.getStream() << "GENNMI_CHECK(gennmi_push_mirrors());" << std::endl;
        if(timing) { funcEnv.getStream() << timerStop("initTime") << std::endl; }
    }
    body << std::endl;

    // column views to build once connectivity is on the device: (merged group index, number of groups)
    std::vector<std::pair<size_t, size_t>> remapGroups;
    body << "void initializeSparse()";
    {
        CodeStream::Scope b(body);
        if(timing) { body << timerStart << std::endl; }
        EnvironmentExternal funcEnv(initEnv);
        funcEnv.add(model.getTimePrecision().addConst(), "dt", Type::writeNumeric(model.getDT(), model.getTimePrecision()));

        std::ostringstream remapStream;
        CodeStream remap(remapStream);
        modelMerged.genMergedSynapseSparseInitGroups(
            *this, memorySpaces,
            [&](auto &s)
            {
                const bool learnPost = s.getArchetype().isPostSpikeRequired() || s.getArchetype().isPostSpikeEventRequired();
                forEachGroup(funcEnv, "SynapseSparseInitGroup", s.getIndex(), s.getGroups().size(), [&]
                {
                    EnvironmentGroupMergedField<SynapseSparseInitGroupMerged> env(funcEnv, s);
                    buildStandardEnvironment(env, batchSize);
                    // (variables initialised from a kernel were written while the rows were built)
                    bool anyRowVar = false;
                    for(const auto &var : s.getArchetype().getWUInitialiser().getSnippet()->getVars()) {
                        const auto &init = s.getArchetype().getWUInitialiser().getVarInitialisers().at(var.name);
                        anyRowVar = anyRowVar || (!Utils::areTokensEmpty(init.getCodeTokens()) && !init.isKernelRequired());
                    }
                    if(emitDeviceVars(s, env, "(size_t)" + env["num_pre"] + " * " + env["_row_stride"])) {
                        // (drawn on the device)
                    }
                    else if(s.getArchetype().isWUVarInitRequired() && anyRowVar) {
                        // (rows the device generated are fetched first)
                        env.printLine("GENNMI_CHECK(gennmi_mirror_ensure_host($(_row_length))); GENNMI_CHECK(gennmi_mirror_ensure_host($(_ind)));");
                        env.print("for(unsigned int i = 0; i < $(num_pre); i++)");
                        CodeStream::Scope loop(env.getStream());
                        env.add(Type::Uint32.addConst(), "id_pre", "i");
                        env.add(Type::Uint32.addConst(), "row_len", "$(_row_length)[i]");
                        s.generateInit(*this, env, batchSize);
                    }
                    if(learnPost && s.getArchetype().getSparseIndType() != Type::Uint32) {
                        unsupported("the column view of projection '" + s.getArchetype().getName() + "' over a narrow sparse index type");
                    }
                    if(learnPost) {
                        // evaluated here so the fields exist; executed after the upload below
                        remap << "for(unsigned int g = 0; g < " << s.getGroups().size() << "; g++)";
                        CodeStream::Scope r(remap);
                        remap << "const auto *group = &mergedSynapseSparseInitGroup" << s.getIndex() << "[g];" << std::endl;
                        remap << "GENNMI_CHECK(gennmi_build_remap(" << env["num_pre"] << ", " << env["num_post"] << ", " << env["_row_stride"] << ", " << env["_col_stride"]
                              << ", gennmiDev(" << env["_row_length"] << "), gennmiDev(" << env["_ind"] << "), gennmiDev(" << env["_col_length"] << "), gennmiDev(" << env["_remap"] << ")));" << std::endl;
                    }
                });
            });
        // per-synapse variables of custom updates over SPARSE matrices: row by row, like the projection's own
        modelMerged.genMergedCustomWUUpdateSparseInitGroups(
            *this, memorySpaces,
            [&](auto &c)
            {
                forEachGroup(funcEnv, "CustomWUUpdateSparseInitGroup", c.getIndex(), c.getGroups().size(), [&]
                {
                    EnvironmentGroupMergedField<CustomWUUpdateSparseInitGroupMerged> env(funcEnv, c);
                    buildStandardEnvironment(env, batchSize);
                    env.printLine("GENNMI_CHECK(gennmi_mirror_ensure_host($(_row_length))); GENNMI_CHECK(gennmi_mirror_ensure_host($(_ind)));");
                    env.print("for(unsigned int i = 0; i < $(num_pre); i++)");
                    CodeStream::Scope loop(env.getStream());
                    env.add(Type::Uint32.addConst(), "id_pre", "i");
                    env.add(Type::Uint32.addConst(), "row_len", "$(_row_length)[i]");
                    c.generateInit(*this, env, batchSize);
                });
            });
        // per-synapse variables of custom connectivity updates
        modelMerged.genMergedCustomConnectivityUpdateSparseInitGroups(
            *this, memorySpaces,
            [&](auto &c)
            {
                forEachGroup(funcEnv, "CustomConnectivityUpdateSparseInitGroup", c.getIndex(), c.getGroups().size(), [&]
                {
                    EnvironmentGroupMergedField<CustomConnectivityUpdateSparseInitGroupMerged> env(funcEnv, c);
                    buildStandardEnvironment(env);
                    env.printLine("GENNMI_CHECK(gennmi_mirror_ensure_host($(_row_length))); GENNMI_CHECK(gennmi_mirror_ensure_host($(_ind)));");
                    env.print("for(unsigned int i = 0; i < $(num_pre); i++)");
                    CodeStream::Scope loop(env.getStream());
                    env.add(Type::Uint32.addConst(), "id_pre", "i");
                    env.add(Type::Uint32.addConst(), "row_len", "$(_row_length)[i]");
                    c.generateInit(*this, env, batchSize);
                });
            });
        funcEnv.getStream() << "GENNMI_CHECK(gennmi_push_mirrors());" << std::endl;
        funcEnv.getStream() << remapStream.str();
        if(timing) { funcEnv.getStream() << "GENNMI_CHECK(gennmi_synchronize());" << std::endl << timerStop("initSparseTime") << std::endl; }
    }

    modelMerged.genMergedNeuronInitGroupStructs(os, *this);
    modelMerged.genMergedSynapseInitGroupStructs(os, *this);
    modelMerged.genMergedSynapseConnectivityInitGroupStructs(os, *this);
    modelMerged.genMergedSynapseSparseInitGroupStructs(os, *this);
    modelMerged.genMergedCustomUpdateInitGroupStructs(os, *this);
    modelMerged.genMergedCustomWUUpdateInitGroupStructs(os, *this);
    modelMerged.genMergedCustomWUUpdateSparseInitGroupStructs(os, *this);
    modelMerged.genMergedCustomConnectivityUpdatePreInitStructs(os, *this);
    modelMerged.genMergedCustomConnectivityUpdatePostInitStructs(os, *this);
    modelMerged.genMergedCustomConnectivityUpdateSparseInitStructs(os, *this);
    modelMerged.genMergedNeuronInitGroupHostStructArrayPush(os, *this);
    modelMerged.genMergedSynapseInitGroupHostStructArrayPush(os, *this);
    modelMerged.genMergedSynapseConnectivityInitGroupHostStructArrayPush(os, *this);
    modelMerged.genMergedSynapseSparseInitGroupHostStructArrayPush(os, *this);
    modelMerged.genMergedCustomUpdateInitGroupHostStructArrayPush(os, *this);
    modelMerged.genMergedCustomWUUpdateInitGroupHostStructArrayPush(os, *this);
    modelMerged.genMergedCustomWUUpdateSparseInitGroupHostStructArrayPush(os, *this);
    modelMerged.genMergedCustomConnectivityUpdatePreInitHostStructArrayPush(os, *this);
    modelMerged.genMergedCustomConnectivityUpdatePostInitHostStructArrayPush(os, *this);
    modelMerged.genMergedCustomConnectivityUpdateSparseInitHostStructArrayPush(os, *this);
    preambleHandler(os);
    os << bodyStream.str();
}
//--------------------------------------------------------------------------
// Loop shapes of the generic initialisation code: plain host loops
//--------------------------------------------------------------------------
void Backend::genPopVariableInit(EnvironmentExternalBase &env, HandlerEnv handler) const
{
    handler(env);
}
void Backend::genVariableInit(EnvironmentExternalBase &env, const std::string &count, const std::string &indexVarName, HandlerEnv handler) const
{
    // a neuron variable the device has just drawn (genInit): its host loop is left out
    if(!m_DeviceInitialisedVars.empty()) {
        std::string target;
        try { target = env["_value"]; } catch(const std::exception&) {}     // (loops that initialise no variable have no such name)
        const size_t arrow = target.rfind("->");
        if(arrow != std::string::npos && m_DeviceInitialisedVars.count(target.substr(arrow + 2))) { return; }
    }
    env.getStream() << "for(unsigned int k = 0; k < (" << env[count] << "); k++)";
    CodeStream::Scope b(env.getStream());
    EnvironmentExternal varEnv(env);
    varEnv.add(Type::Uint32, indexVarName, "k");
    handler(varEnv);
}
void Backend::genSparseSynapseVariableRowInit(EnvironmentExternalBase &env, HandlerEnv handler) const
{
    env.print("for(unsigned int j = 0; j < $(_row_length)[$(id_pre)]; j++)");
    CodeStream::Scope b(env.getStream());
    EnvironmentExternal varEnv(env);
    varEnv.add(Type::Uint32, "id_syn", "idSyn", {varEnv.addInitialiser("const unsigned int idSyn = ($(id_pre) * $(_row_stride)) + j;")});
    varEnv.add(Type::Uint32, "id_post", "idPost", {varEnv.addInitialiser("const unsigned int idPost = $(_ind)[$(id_syn)];")});
    handler(varEnv);
}
void Backend::genDenseSynapseVariableRowInit(EnvironmentExternalBase &env, HandlerEnv handler) const
{
    env.print("for(unsigned int j = 0; j < $(num_post); j++)");
    CodeStream::Scope b(env.getStream());
    EnvironmentExternal varEnv(env);
    varEnv.add(Type::Uint32, "id_syn", "idSyn", {varEnv.addInitialiser("const unsigned int idSyn = ($(id_pre) * $(_row_stride)) + j;")});
    varEnv.add(Type::Uint32, "id_post", "j");
    handler(varEnv);
}
void Backend::genKernelSynapseVariableInit(EnvironmentExternalBase &env, SynapseInitGroupMerged &sg, HandlerEnv handler) const
{
    // one nested loop per kernel dimension, innermost last; id_syn is the row-major kernel index
    EnvironmentExternal loopEnv(env);
    const size_t numDims = sg.getArchetype().getKernelSize().size();
    std::string index;
    for(size_t d = 0; d < numDims; d++) {
        const std::string v = "k" + std::to_string(d);
        loopEnv.getStream() << "for(unsigned int " << v << " = 0; " << v << " < " << getKernelSize(sg, d) << "; " << v << "++)" << CodeStream::OB(500 + d);
        loopEnv.add(Type::Uint32.addConst(), "id_kernel_" + std::to_string(d), v);
        index = index.empty() ? v : ("(" + index + ") * " + getKernelSize(sg, d) + " + " + v);
    }
    {
        EnvironmentExternal varEnv(static_cast<EnvironmentExternalBase&>(loopEnv));
        varEnv.add(Type::Uint32.addConst(), "id_syn", "idSyn", {varEnv.addInitialiser("const unsigned int idSyn = " + index + ";")});
        handler(varEnv);
    }
    for(size_t d = numDims; d > 0; d--) {
        loopEnv.getStream() << CodeStream::CB(500 + d - 1);
    }
}
void Backend::genKernelCustomUpdateVariableInit(EnvironmentExternalBase &env, CustomWUUpdateInitGroupMerged &cu, HandlerEnv handler) const
{
    // the same nest of loops over the kernel's dimensions as for a projection's own kernel variables
    EnvironmentExternal loopEnv(env);
    const size_t numDims = cu.getArchetype().getSynapseGroup()->getKernelSize().size();
    std::string index;
    for(size_t d = 0; d < numDims; d++) {
        const std::string v = "k" + std::to_string(d);
        loopEnv.getStream() << "for(unsigned int " << v << " = 0; " << v << " < " << getKernelSize(cu, d) << "; " << v << "++)" << CodeStream::OB(600 + d);
        loopEnv.add(Type::Uint32.addConst(), "id_kernel_" + std::to_string(d), v);
        index = index.empty() ? v : ("(" + index + ") * " + getKernelSize(cu, d) + " + " + v);
    }
    {
        EnvironmentExternal varEnv(static_cast<EnvironmentExternalBase&>(loopEnv));
        varEnv.add(Type::Uint32.addConst(), "id_syn", "idSyn", {varEnv.addInitialiser("const unsigned int idSyn = " + index + ";")});
        handler(varEnv);
    }
    for(size_t d = numDims; d > 0; d--) {
        loopEnv.getStream() << CodeStream::CB(600 + d - 1);
    }
}
//--------------------------------------------------------------------------
size_t Backend::getSynapticMatrixRowStride(const SynapseGroupInternal &sg) const
{
    if(sg.getMatrixType() & SynapseMatrixConnectivity::SPARSE) {
        // rows padded to 4 entries start on 16-byte boundaries, which the row loads of the kernels exploit
        return padSize(sg.getMaxConnections(), 4);
    }
    else if(sg.getMatrixType() & SynapseMatrixConnectivity::PROCEDURAL) {
        // The stride the same snippet would give a stored matrix (the reference only evaluates calcMaxRowLength for SPARSE
        // groups, synapseGroup.cc:420-430): the regenerated weights are indexed by row * stride + position like stored ones.
        const auto &init = sg.getSparseConnectivityInitialiser();
        const auto calcMaxRowLength = init.getSnippet()->getCalcMaxRowLengthFunc();
        return calcMaxRowLength ? calcMaxRowLength(sg.getSrcNeuronGroup()->getNumNeurons(), sg.getTrgNeuronGroup()->getNumNeurons(), init.getParams())
                                : sg.getMaxConnections();
    }
    else if(sg.getMatrixType() & SynapseMatrixConnectivity::TOEPLITZ) {
        return sg.getMaxConnections();
    }
    else if(sg.getMatrixType() & SynapseMatrixConnectivity::BITMASK) {
        return padSize(sg.getTrgNeuronGroup()->getNumNeurons(), 32);
    }
    else {
        return sg.getTrgNeuronGroup()->getNumNeurons();
    }
}
//--------------------------------------------------------------------------
void Backend::genDefinitionsPreamble(CodeStream &os, const ModelSpecMerged&) const
{
    os << "// Standard C++ includes" << std::endl;
    for(const char *h : {"algorithm", "cassert", "chrono", "cmath", "cstdint", "cstring", "iostream", "random", "stdexcept", "string", "vector"}) {
        os << "#include <" << h << ">" << std::endl;
    }
    os << std::endl;
    os << "// MI355X device library" << std::endl;
    os << "#include \"genn_mi355x.h\"" << std::endl;
    if(hasDeviceModules()) {
        os << "// building blocks of the generated kernels: seen by the device pass of a module only (hipcc --genco); the host" << std::endl;
        os << "// pass (the host compiler) sees structs and host functions, which reach the device through the C ABI above" << std::endl;
        os << "#ifdef __HIPCC__" << std::endl;
        os << "#include \"genn_mi355x_kernel_support.h\"" << std::endl;
        os << "#endif" << std::endl;
        os << "extern bool gennmiStructsDirty;" << std::endl;
        os << "extern gennmi_program *gennmiProgram;" << std::endl;
        os << "extern uint32_t *gennmiProgramError;" << std::endl;
        os << "void gennmiUploadCustomUpdateGroups();" << std::endl;
        os << "void gennmiFreeCustomUpdateGroups();" << std::endl;
    }
    if(m_GeneratedKernels) {
        os << "void gennmiUploadNeuronGroups();" << std::endl;
        os << "void gennmiUploadSynapseGroups();" << std::endl;
        os << "void gennmiFreeNeuronGroups();" << std::endl;
        os << "void gennmiFreeSynapseGroups();" << std::endl;
    }
    os << "#define GENNMI_CHECK(call) do { if((call) != GENNMI_OK) { throw std::runtime_error(std::string(__FILE__) + \": \" + std::to_string(__LINE__) + \": \" + gennmi_last_error()); } } while(0)" << std::endl;
    os << std::endl;
    os << "extern gennmi_runner *gennmiRunner;" << std::endl;
    os << "void gennmiBuildNeuronGroups();" << std::endl;
    os << "void gennmiBuildSynapseGroups();" << std::endl;
    os << "void gennmiEnsureFinalised();" << std::endl;
    os << "uint32_t *gennmiScratch(size_t count);" << std::endl;
    os << "// merged groups hold host pointers; kernels need the device buffers registered behind them" << std::endl;
    os << "template<typename T> inline T *gennmiDev(T *host)";
    {
        CodeStream::Scope b(os);
        os << "void *dev = nullptr;" << std::endl;
        os << "GENNMI_CHECK(gennmi_mirror_device_pointer((const void*)host, &dev));" << std::endl;
        os << "return (T*)dev;" << std::endl;
    }
    os << "using std::min;" << std::endl;
    os << "using std::max;" << std::endl;
    os << "// seed of device-side initialisation for models that leave theirs at 0 (a different one every run, ModelSpec::setSeed)" << std::endl;
    os << "inline uint64_t gennmiRandomSeed() { static const uint64_t seed = [] { std::random_device rd; return ((uint64_t)rd() << 32) | rd(); }(); return seed; }" << std::endl;
    os << std::endl;
}
//--------------------------------------------------------------------------
void Backend::genRunnerPreamble(CodeStream &os, const ModelSpecMerged&) const
{
    os << "gennmi_runner *gennmiRunner = nullptr;" << std::endl;
    if(hasDeviceModules()) {
        os << "// the model's generated device code: code objects, launch sequences, stream, timers and error flag live in the device library" << std::endl;
        os << "gennmi_program *gennmiProgram = nullptr;" << std::endl;
        os << "uint32_t *gennmiProgramError = nullptr;" << std::endl;
    }
    os << "static bool gennmiFinalised = false;" << std::endl;
    os << "static std::vector<void*> gennmiScratchBuffers;" << std::endl;
    os << "uint32_t *gennmiScratch(size_t count)";
    {
        CodeStream::Scope b(os);
        os << "void *p = nullptr;" << std::endl;
        os << "GENNMI_CHECK(gennmi_malloc(&p, count * sizeof(uint32_t)));" << std::endl;
        os << "GENNMI_CHECK(gennmi_memset(p, 0, count * sizeof(uint32_t)));" << std::endl;
        os << "gennmiScratchBuffers.push_back(p);" << std::endl;
        os << "return (uint32_t*)p;" << std::endl;
    }
    if(m_GeneratedKernels) {
        os << "// device copies of the merged-group struct arrays: uploaded before the first step and after every push of a dynamic field" << std::endl;
        os << "bool gennmiStructsDirty = true;" << std::endl;
        os << "void gennmiBuildNeuronGroups() {}" << std::endl;
        os << "void gennmiBuildSynapseGroups() {}" << std::endl;
        os << "void gennmiEnsureFinalised()";
        {
            CodeStream::Scope b(os);
            os << "if(!gennmiStructsDirty) { return; }" << std::endl;
            os << "GENNMI_CHECK(gennmi_synchronize());" << std::endl;
            os << "gennmiUploadSynapseGroups();" << std::endl;     // (first: the neuron update walks the ring-pointer groups this uploads)
            os << "gennmiUploadNeuronGroups();" << std::endl;
            os << "gennmiUploadCustomUpdateGroups();" << std::endl;
            os << "gennmiStructsDirty = false;" << std::endl;
            os << "gennmiFinalised = true;" << std::endl;
        }
        os << std::endl;
        return;
    }
    if(m_CustomUpdateKernels) {
        os << "// device copies of the custom updates' merged-group struct arrays: uploaded before the first use and after every push of a dynamic field" << std::endl;
        os << "bool gennmiStructsDirty = true;" << std::endl;
    }
    os << "// every merged update group becomes descriptors of the device library, once, before the first step" << std::endl;
    os << "void gennmiEnsureFinalised()";
    {
        CodeStream::Scope b(os);
        if(m_CustomUpdateKernels) {
            os << "if(gennmiStructsDirty) { GENNMI_CHECK(gennmi_synchronize()); gennmiUploadCustomUpdateGroups(); gennmiStructsDirty = false; }" << std::endl;
        }
        os << "if(gennmiFinalised) { return; }" << std::endl;
        os << "gennmiBuildNeuronGroups();" << std::endl;
        os << "gennmiBuildSynapseGroups();" << std::endl;
        if(getPreferences<Preferences>().orderedAccumulation) {
            os << "GENNMI_CHECK(gennmi_runner_set_ordered(gennmiRunner, 1));" << std::endl;
        }
        os << "GENNMI_CHECK(gennmi_runner_finalise(gennmiRunner));" << std::endl;
        if(getPreferences<Preferences>().stepQueueLength > 0) {
            os << "GENNMI_CHECK(gennmi_runner_set_step_queue(gennmiRunner, " << getPreferences<Preferences>().stepQueueLength << "u));" << std::endl;
        }
        os << "gennmiFinalised = true;" << std::endl;
    }
    os << std::endl;
}
//--------------------------------------------------------------------------
void Backend::genAllocateMemPreamble(CodeStream &os, const ModelSpecMerged &modelMerged) const
{
    const ModelSpecInternal &model = modelMerged.getModel();
    os << "GENNMI_CHECK(gennmi_init(" << getPreferences<Preferences>().deviceID << "));" << std::endl;
    if(hasDeviceModules()) { os << "gennmiStructsDirty = true;" << std::endl; }
    if(!m_GeneratedKernels) {
        os << "GENNMI_CHECK(gennmi_runner_create(&gennmiRunner, " << Type::writeNumeric(model.getDT(), model.getTimePrecision()) << ", " << model.getBatchSize() << "u));" << std::endl;
        if(model.isTimingEnabled()) {
            os << "GENNMI_CHECK(gennmi_runner_set_timing(gennmiRunner, 1));" << std::endl;
        }
    }
    if(hasDeviceModules()) {
        // (generated step kernels: updateSynapses / updateNeurons calls are noted and replayed from a captured graph of
        // stepQueueLength steps; custom updates beside library kernels are launched when called, on the runner's stream)
        os << "GENNMI_CHECK(gennmi_program_create(&gennmiProgram, gennmiRunner, " << (m_GeneratedKernels ? getPreferences<Preferences>().stepQueueLength : 0u) << "u));" << std::endl;
        os << "GENNMI_CHECK(gennmi_program_error_flag(gennmiProgram, &gennmiProgramError));" << std::endl;
        if(model.isTimingEnabled()) {
            os << "GENNMI_CHECK(gennmi_program_set_timing(gennmiProgram, 1));" << std::endl;
        }
    }
}
//--------------------------------------------------------------------------
void Backend::genFreeMemPreamble(CodeStream &os, const ModelSpecMerged&) const
{
    if(hasDeviceModules()) {
        os << "if(gennmiProgram) { GENNMI_CHECK(gennmi_program_destroy(gennmiProgram)); gennmiProgram = nullptr; gennmiProgramError = nullptr; }" << std::endl;
        os << "gennmiFreeCustomUpdateGroups();" << std::endl;
        if(m_GeneratedKernels) { os << "gennmiFreeNeuronGroups();" << std::endl << "gennmiFreeSynapseGroups();" << std::endl; }
    }
    os << "if(gennmiRunner) { GENNMI_CHECK(gennmi_runner_destroy(gennmiRunner)); gennmiRunner = nullptr; }" << std::endl;
    os << "for(void *p : gennmiScratchBuffers) { gennmi_free(p); }" << std::endl;
    os << "gennmiScratchBuffers.clear();" << std::endl;
    os << "gennmiFinalised = false;" << std::endl;
}
//--------------------------------------------------------------------------
void Backend::genStepTimeFinalisePreamble(CodeStream &os, const ModelSpecMerged &modelMerged) const
{
    if(m_GeneratedKernels) {
        // (the timers are read right after this: genTimer.  A bounded wait that expired in a kernel is reported by this call, and —
        // whatever the timing setting — by every later call of the library that waits for the device: pulls, synchronisation)
        if(modelMerged.getModel().isTimingEnabled()) {
            os << "GENNMI_CHECK(gennmi_program_synchronize(gennmiProgram));" << std::endl;
        }
        return;
    }
    // the reference's device backends synchronise here too when timing (backendCUDAHIP.cc:1400-1411)
    if(modelMerged.getModel().isTimingEnabled()) {
        os << "GENNMI_CHECK(gennmi_runner_synchronize(gennmiRunner));" << std::endl;
        os << "GENNMI_CHECK(gennmi_runner_get_times(gennmiRunner, &neuronUpdateTime, &presynapticUpdateTime, &postsynapticUpdateTime));" << std::endl;
    }
}
//--------------------------------------------------------------------------
std::string State::getDeviceName() const
{
    char name[256] = {0};
    if(gennmi_device_name(name, sizeof(name)) != GENNMI_OK) { throw std::runtime_error(gennmi_last_error()); }
    return name;
}
size_t State::getFreeDeviceMemBytes() const
{
    size_t bytes = 0;
    if(gennmi_free_device_memory_bytes(&bytes) != GENNMI_OK) { throw std::runtime_error(gennmi_last_error()); }
    return bytes;
}
void State::synchronize() const
{
    if(gennmi_synchronize() != GENNMI_OK) { throw std::runtime_error(gennmi_last_error()); }
}
std::unique_ptr<GeNN::Runtime::StateBase> Backend::createState(const Runtime::Runtime&) const
{
    return std::make_unique<State>();
}
void Backend::genPushProfilerRange(CodeStream &os, const std::string &name) const
{
    if(getPreferences<Preferences>().profilerRanges) {
        os << "gennmi_profiler_range_push(\"" << name << "\");" << std::endl;
    }
}
void Backend::genPopProfilerRange(CodeStream &os) const
{
    if(getPreferences<Preferences>().profilerRanges) {
        os << "gennmi_profiler_range_pop();" << std::endl;
    }
}
std::unique_ptr<Runtime::ArrayBase> Backend::createArray(const Type::ResolvedType &type, size_t count,
                                                         VarLocation location, bool uninitialized) const
{
    return std::make_unique<Array>(type, count, location, uninitialized);
}
std::unique_ptr<Runtime::ArrayBase> Backend::createPopulationRNG(size_t) const
{
    return std::unique_ptr<Runtime::ArrayBase>();
}
//--------------------------------------------------------------------------
// Extra global parameters allocated from generated host code (initializeHost): plain host arrays
//--------------------------------------------------------------------------
void Backend::genLazyVariableDynamicAllocation(CodeStream &os, const Type::ResolvedType &type, const std::string &name,
                                               VarLocation, const std::string &countVarName) const
{
    const auto &valueType = type.isPointer() ? *type.getPointer().valueType : type;
    os << (type.isPointer() ? "*" : "") << "$(_" << name << ") = new " << valueType.getValue().name << "[" << countVarName << "];" << std::endl;
}
// (pointer-typed: an extra global parameter of host initialisation code, a plain host array — nothing to copy.  Otherwise: an
// array of a custom connectivity update's host update code, whose host buffer has a device buffer registered behind it)
void Backend::genLazyVariableDynamicPush(CodeStream &os, const Type::ResolvedType &type, const std::string &name, VarLocation, const std::string &countVarName) const
{
    if(type.isPointer()) { return; }
    os << "GENNMI_CHECK(gennmi_memcpy_to_device(gennmiDev($(_" << name << ")), $(_" << name << "), (size_t)(" << countVarName << ") * sizeof(" << type.getName() << ")));" << std::endl;
}
void Backend::genLazyVariableDynamicPull(CodeStream &os, const Type::ResolvedType &type, const std::string &name, VarLocation, const std::string &countVarName) const
{
    if(type.isPointer()) { return; }
    os << "GENNMI_CHECK(gennmi_memcpy_from_device($(_" << name << "), gennmiDev($(_" << name << ")), (size_t)(" << countVarName << ") * sizeof(" << type.getName() << ")));" << std::endl;
}
void Backend::genMergedDynamicVariablePush(CodeStream &os, const std::string &suffix, size_t mergedGroupIdx,
                                           const std::string &groupIdx, const std::string &fieldName,
                                           const std::string &egpName) const
{
    os << "merged" << suffix << "Group" << mergedGroupIdx << "[" << groupIdx << "]." << fieldName << " = " << egpName << ";" << std::endl;
    if(hasDeviceModules()) { os << "gennmiStructsDirty = true;" << std::endl; }
}
//--------------------------------------------------------------------------
std::string Backend::getAtomicOperation(const std::string &lhsPointer, const std::string &rhsValue,
                                        const Type::ResolvedType&, AtomicOperation op) const
{
    // only host-side initialisation code is generated, and it is single-threaded
    return "(*(" + lhsPointer + ") " + ((op == AtomicOperation::ADD) ? "+=" : "|=") + " (" + rhsValue + "))";
}
void Backend::genGlobalDeviceRNG(CodeStream&, CodeStream&, CodeStream&, CodeStream&) const
{
    unsupported("a device random number generator");
}
void Backend::genTimer(CodeStream &definitions, CodeStream &runner, CodeStream &allocations, CodeStream &free,
                       CodeStream &stepTimeFinalise, const std::string &name, bool updateInStepTime) const
{
    // library kernels: durations are accumulated inside the device library (gennmi_runner_set_timing / get_times);
    // initialisation: wall-clock time of the host functions (genInit)
    // (beside library kernels only the custom updates' kernels are generated, and timed this way)
    if(!hasDeviceModules() || name == "init" || name == "initSparse" || (!m_GeneratedKernels && name.rfind("customUpdate", 0) != 0)) { return; }
    // generated kernels: the device library records a pair of events around each launch of the update's kind, as the
    // reference's device backends do inline (backendCUDAHIP.cc:1479-1504), and accumulates their durations per timer
    (void)definitions; (void)runner; (void)allocations; (void)free;
    if(updateInStepTime) {
        stepTimeFinalise << "GENNMI_CHECK(gennmi_program_get_time(gennmiProgram, " << timerId(name) << ", &" << name << "Time));" << std::endl;
    }
}
// which of the program's timers accumulates an update's launches (asked for by the modules that register the launches and by
// the runner that reads the time)
int Backend::timerId(const std::string &name) const
{
    const auto it = m_TimerIds.find(name);
    if(it != m_TimerIds.cend()) { return it->second; }
    if(m_TimerIds.size() >= GENNMI_MAX_TIMERS) { unsupported("this many timed update groups"); }
    const int id = (int)m_TimerIds.size();
    m_TimerIds.emplace(name, id);
    return id;
}
void Backend::genReturnFreeDeviceMemoryBytes(CodeStream &os) const
{
    os << "size_t freeBytes = 0;" << std::endl;
    os << "GENNMI_CHECK(gennmi_free_device_memory_bytes(&freeBytes));" << std::endl;
    os << "return freeBytes;" << std::endl;
}
void Backend::genAssert(CodeStream &os, const std::string &condition) const
{
    os << "assert(" << condition << ");" << std::endl;
}
//--------------------------------------------------------------------------
// Build system: the runner is host C++ linked against the device library
//--------------------------------------------------------------------------
void Backend::genMakefilePreamble(std::ostream &os) const
{
    std::string root = getPreferences<Preferences>().installRoot;
    if(root.empty()) {
        const char *env = std::getenv("GENN_MI355X_ROOT");
        root = env ? env : GENNMI_DEFAULT_ROOT;
    }
    std::string cxxFlags = "-c -fPIC -std=c++17 -MMD -MP -I\"" + root + "/include\" " + getPreferences().userCxxFlagsGNU;
    cxxFlags += getPreferences().debugCode ? " -O0 -g" : " -O2";
    os << "CXXFLAGS := " << cxxFlags << std::endl;
    if(hasDeviceModules()) {
        // modules that hold device code are compiled a second time, device side only, into a gfx950 code object: fp32 operations
        // neither contracted nor packed so that results match the SingleThreadedCPU backend's operation for operation
        os << "HIPCC := " << (std::getenv("HIP_PATH") ? std::string(std::getenv("HIP_PATH")) + "/bin/hipcc" : std::string("hipcc")) << std::endl;
        os << "HIPCCFLAGS := --genco --offload-arch=gfx950 -std=c++17 -x hip -I\"" << root << "/include\" " << (getPreferences().debugCode ? "-O0 -g" : "-O2")
           << " -ffp-contract=off -Xclang -target-feature -Xclang -packed-fp32-ops -Wno-unused-value" << std::endl;
    }
    os << "LINKFLAGS := -shared" << std::endl;
    os << "LINKLIBS := -L\"" << root << "/genn_amd/lib\" -lgenn_mi355x -Wl,-rpath,\"" << root << "/genn_amd/lib\"" << std::endl;
    os << std::endl;
}
void Backend::genMakefileLinkRule(std::ostream &os) const
{
    os << "\t@$(CXX) $(LINKFLAGS) -o $@ $(OBJECTS) $(LINKLIBS)" << std::endl;
}
void Backend::genMakefileCompileRule(std::ostream &os) const
{
    os << "%.o: %.cc %.d" << std::endl;
    if(!hasDeviceModules()) {
        os << "\t@$(CXX) $(CXXFLAGS) -o $@ $<" << std::endl;
        return;
    }
    // host pass into <module>.host.o; for a module that says GENNMI_DEVICE_MODULE, device pass into <module>.hsaco, which is
    // wrapped into an object (symbols gennmi_<module>_image / _image_end) and joined with the host object into <module>.o
    os << "\t@$(CXX) $(CXXFLAGS) -MF $*.d -MT $@ -o $*.host.o $<" << std::endl;
    os << "\t@if grep -q '^#define GENNMI_DEVICE_MODULE' $<; then \\" << std::endl;
    os << "\t    $(HIPCC) $(HIPCCFLAGS) -o $*.hsaco $< && \\" << std::endl;
    os << "\t    printf '.section .rodata\\n.balign 4096\\n.global gennmi_$*_image\\ngennmi_$*_image:\\n.incbin \"$*.hsaco\"\\n.global gennmi_$*_image_end\\ngennmi_$*_image_end:\\n.section .note.GNU-stack,\"\",@progbits\\n' > $*.image.s && \\" << std::endl;
    os << "\t    $(CXX) -c -o $*.image.o $*.image.s && $(LD) -r -o $@ $*.host.o $*.image.o; \\" << std::endl;
    os << "\telse cp $*.host.o $@; fi" << std::endl;
}
void Backend::genNMakefilePreamble(std::ostream&) const { unsupported("NMake"); }
void Backend::genNMakefileLinkRule(std::ostream&) const { unsupported("NMake"); }
void Backend::genNMakefileCompileRule(std::ostream&) const { unsupported("NMake"); }
void Backend::genMSBuildConfigProperties(std::ostream&) const {}
void Backend::genMSBuildImportProps(std::ostream&) const {}
void Backend::genMSBuildItemDefinitions(std::ostream&) const {}
void Backend::genMSBuildCompileModule(const std::string&, std::ostream&) const {}
void Backend::genMSBuildImportTarget(std::ostream&) const {}
//--------------------------------------------------------------------------
bool Backend::isGlobalHostRNGRequired(const ModelSpecInternal &model) const
{
    // initialisation runs on the host, so any random initialisation draws from the host generator
    const auto &ngs = model.getNeuronGroups();
    const auto &sgs = model.getSynapseGroups();
    return std::any_of(ngs.cbegin(), ngs.cend(), [](const auto &n){ return n.second.isInitRNGRequired(); })
        || std::any_of(sgs.cbegin(), sgs.cend(), [](const auto &s){ return s.second.isWUInitRNGRequired() || s.second.getSparseConnectivityInitialiser().isRNGRequired()
                                                                          || s.second.getSparseConnectivityInitialiser().isHostRNGRequired(); })
        || std::any_of(model.getCustomUpdates().cbegin(), model.getCustomUpdates().cend(), [](const auto &c){ return c.second.isInitRNGRequired(); })
        || std::any_of(model.getCustomWUUpdates().cbegin(), model.getCustomWUUpdates().cend(), [](const auto &c){ return c.second.isInitRNGRequired(); })
        || std::any_of(model.getCustomConnectivityUpdates().cbegin(), model.getCustomConnectivityUpdates().cend(),
                       [](const auto &c){ return Utils::isRNGRequired(c.second.getVarInitialisers()) || Utils::isRNGRequired(c.second.getPreVarInitialisers())
                                                 || Utils::isRNGRequired(c.second.getPostVarInitialisers()) || Utils::isRNGRequired(c.second.getHostUpdateCodeTokens()); });
}
size_t Backend::getDeviceMemoryBytes() const
{
    size_t bytes = 0;
    return (gennmi_free_device_memory_bytes(&bytes) == GENNMI_OK) ? bytes : 0;
}
boost::uuids::detail::sha1::digest_type Backend::getHashDigest() const
{
    boost::uuids::detail::sha1 hash;
    Utils::updateHash("MI355X", hash);
    getPreferences<Preferences>().updateHash(hash);
    return hash.get_digest();
}
//--------------------------------------------------------------------------
// GeNN::CodeGenerator::MI355X::Optimiser
//--------------------------------------------------------------------------
namespace Optimiser
{
Backend createBackend(const ModelSpecInternal &model, const filesystem::path&, plog::Severity backendLevel,
                      plog::IAppender *backendAppender, const Preferences &preferences)
{
    if(plog::get<Logging::CHANNEL_BACKEND>() == nullptr) {
        plog::init<Logging::CHANNEL_BACKEND>(backendLevel, backendAppender);
    }
    else {
        plog::get<Logging::CHANNEL_BACKEND>()->setMaxSeverity(backendLevel);
    }
    bool generated = (preferences.kernelSource == Preferences::KernelSource::GENERATED);
    if(preferences.kernelSource == Preferences::KernelSource::AUTO) {
        // generated kernels when some snippet of the model is not one the device library implements ...
        auto recognised = [](auto fn) { try { fn(); return true; } catch(const std::runtime_error&) { return false; } };
        for(const auto &n : model.getNeuronGroups()) {
            generated = generated || !recognised([&]{ recogniseNeuron(n.second.getModel(), n.first); });
            for(const auto *cs : n.second.getCurrentSources()) {
                const std::string code = cs->getModel()->getInjectionCode();
                const bool known = same(code, CurrentSourceModels::DC::getInstance()->getInjectionCode()) || same(code, CurrentSourceModels::PoissonExp::getInstance()->getInjectionCode())
                                   || (same(code, "injectCurrent(noise[id]);") && cs->getModel()->getExtraGlobalParams().size() == 1);
                generated = generated || !known;
            }
        }
        for(const auto &s : model.getSynapseGroups()) {
            generated = generated || !recognised([&]{ recognisePSM(s.second.getPSInitialiser().getSnippet(), s.first); });
            generated = generated || !recognised([&]{ recogniseWUM(s.second.getWUInitialiser().getSnippet(), s.first); });
            // ... or when a learning rule meets delay slots (spike times, traces and weight-update variables per slot): the
            // library's plastic kernels read populations without a ring, GeNN's generic code in generated kernels handles it
            const auto *wum = s.second.getWUInitialiser().getSnippet();
            const bool learns = !wum->getPostSpikeSynCode().empty() || !wum->getPreSpikeCode().empty() || !wum->getPostSpikeCode().empty()
                                || !wum->getPreVars().empty() || !wum->getPostVars().empty();
            const bool delayed = s.second.getSrcNeuronGroup()->isDelayRequired() || s.second.getTrgNeuronGroup()->isDelayRequired()
                                 || s.second.getBackPropDelaySteps() != 0;
            generated = generated || (learns && delayed);
        }
        // ... or when a parameter is dynamic: the library's descriptors hold parameters as constants, generated kernels read
        // them from the merged structs that setDynamicParamValue rewrites
        auto anyDynamic = [](const auto &params, auto isDynamic)
        {
            return std::any_of(params.cbegin(), params.cend(), [&](const auto &p) { return isDynamic(p.name); });
        };
        for(const auto &n : model.getNeuronGroups()) {
            generated = generated || anyDynamic(n.second.getModel()->getParams(), [&](const std::string &p) { return n.second.isParamDynamic(p); });
            for(const auto *cs : n.second.getCurrentSources()) {
                generated = generated || anyDynamic(cs->getModel()->getParams(), [&](const std::string &p) { return cs->isParamDynamic(p); });
            }
        }
        for(const auto &s : model.getSynapseGroups()) {
            generated = generated || anyDynamic(s.second.getPSInitialiser().getSnippet()->getParams(), [&](const std::string &p) { return s.second.isPSParamDynamic(p); });
            generated = generated || anyDynamic(s.second.getWUInitialiser().getSnippet()->getParams(), [&](const std::string &p) { return s.second.isWUParamDynamic(p); });
        }
        // ... or when a SPARSE projection stores its targets in a narrow type (ModelSpec::setDefaultNarrowSparseIndEnabled): the library
        // reads 32-bit ones, generated code takes the type from the merged struct
        for(const auto &s : model.getSynapseGroups()) {
            generated = generated || ((s.second.getMatrixType() & SynapseMatrixConnectivity::SPARSE) && s.second.getSparseIndType() != Type::Uint32);
        }
        // ... or when the model is not single precision: the library's kernels are fp32
        generated = generated || model.getPrecision() != Type::Float || model.getTimePrecision() != Type::Float;
        // ... or when custom connectivity updates rewire a projection: the library's launch plans rely on rows sorted by target,
        // which removing and adding synapses does not keep
        generated = generated || !model.getCustomConnectivityUpdates().empty();
        if(generated) { LOGI_BACKEND << "The model uses snippets or combinations the device library does not implement, or dynamic parameters: the step's kernels are generated from the model's code"; }
    }
    if(generated && preferences.orderedAccumulation) {
        throw std::runtime_error("MI355X backend: ordered accumulation is a mode of the device library's kernels, not of generated ones");
    }
    // custom updates are arbitrary model code: their kernels are generated whichever kernels the step runs on
    const bool customUpdates = !model.getCustomUpdates().empty() || !model.getCustomWUUpdates().empty() || !model.getCustomConnectivityUpdates().empty();
    return Backend(preferences, generated, customUpdates);
}
}   // namespace Optimiser
}   // namespace GeNN::CodeGenerator::MI355X
