// GeNN::CodeGenerator::MI355X::Backend (see backend.h for the division of labour).
#include "backend.h"
#include "optimiser.h"

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
// Array: a host buffer (always present: generated initialisation code and merged groups work on host pointers)
// mirrored by a device buffer; the pair is registered with the device library so generated code can translate
// pointers.  Counterpart of the Array classes of the reference's backends (hip/backend.cc:61-236).
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
        auto *host = static_cast<std::byte*>(std::calloc(getSizeBytes(), 1));
        if(!host) { throw std::bad_alloc(); }
        setHostPointer(host);
        check(gennmi_malloc(&m_Device, getSizeBytes()), "array allocation");
        check(gennmi_memset(m_Device, 0, getSizeBytes()), "array clear");
        check(gennmi_register_mirror(host, m_Device, getSizeBytes()), "array registration");
    }
    virtual void free() final
    {
        check(gennmi_unregister_mirror(getHostPointer()), "array deregistration");
        check(gennmi_free(m_Device), "array release");
        std::free(getHostPointer());
        m_Device = nullptr;
        setHostPointer(nullptr);
        setCount(0);
    }
    virtual void pushToDevice() final { pushSlice1DToDevice(0, getCount()); }
    virtual void pullFromDevice() final { pullSlice1DFromDevice(0, getCount()); }
    virtual void pushSlice1DToDevice(size_t offset, size_t count) final
    {
        const auto [o, b] = slice(offset, count);
        check(gennmi_memcpy_to_device(static_cast<char*>(m_Device) + o, getHostPointer() + o, b), "push");
    }
    virtual void pullSlice1DFromDevice(size_t offset, size_t count) final
    {
        const auto [o, b] = slice(offset, count);
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

    void *m_Device;
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
unsigned int recogniseWUM(const WeightUpdateModels::Base *m, const std::string &name)
{
    const bool plain = m->getPostSpikeSynCode().empty() && m->getSynapseDynamicsCode().empty() && m->getPreEventSynCode().empty()
                       && m->getPostEventSynCode().empty() && m->getPreSpikeCode().empty() && m->getPostSpikeCode().empty()
                       && m->getPreDynamicsCode().empty() && m->getPostDynamicsCode().empty();
    if(plain && same(m->getPreSpikeSynCode(), WeightUpdateModels::StaticPulse::getInstance()->getPreSpikeSynCode())
       && m->getVars().size() == 1) { return GENNMI_WUM_STATIC_PULSE; }
    if(plain && same(m->getPreSpikeSynCode(), WeightUpdateModels::StaticPulseDendriticDelay::getInstance()->getPreSpikeSynCode())) {
        return GENNMI_WUM_STATIC_PULSE_DENDRITIC_DELAY;
    }
    if(isTraceSTDP(m)) { return GENNMI_WUM_STDP_TRACE; }
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
