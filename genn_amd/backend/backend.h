#pragma once
// GeNN::CodeGenerator::MI355X::Backend — plugs the MI355X device library (include/genn_mi355x.h) into GeNN's code
// generator as one more backend (interface: include/genn/genn/code_generator/backendBase.h:127-486; selected like
// include/genn/backends/single_threaded_cpu/backend.h or hip/backend.h).
//
// Division of labour:
//  * initialize() / initializeSparse() are the reference's own host-side initialisation code, generated through
//    the generic *InitGroupMerged::generateInit machinery, running on the arrays' host buffers; every buffer is then
//    uploaded.  Runtime hands merged groups HOST pointers because isArrayDeviceObjectRequired() is false.
//  * updateSynapses() / updateNeurons() do not run generated model code: each merged update group is recognised as
//    one of the models the device library implements and translated, once, into a descriptor
//    (gennmi_*_update_group_t); anything else is rejected at code-generation time with std::runtime_error.
#include <memory>
#include <map>
#include <set>
#include <string>

#include "backendExport.h"
#include "code_generator/backendBase.h"
#include "code_generator/environment.h"

namespace filesystem { class path; }

namespace GeNN::CodeGenerator::MI355X
{
struct Preferences : public PreferencesBase
{
    //! HIP device ordinal handed to gennmi_init() by the generated allocateMem()
    int deviceID = 0;

    //! Where the generated Makefile finds genn_mi355x.h and libgenn_mi355x.so
    //! (empty: the GENN_MI355X_ROOT environment variable at code-generation time)
    std::string installRoot;

    //! Where the step's device code comes from.  LIBRARY: every neuron, postsynaptic, current-source and weight-update model
    //! must be one the device library implements (anything else is refused); the runner is host code.  GENERATED: kernels
    //! are generated from the model's own code strings for every group and compiled with hipcc into the runner.  AUTO:
    //! LIBRARY when every snippet of the model is recognised, GENERATED otherwise.
    enum class KernelSource { AUTO, LIBRARY, GENERATED };
    KernelSource kernelSource = KernelSource::AUTO;

    //! Validation mode of the device library: synaptic input is summed per postsynaptic neuron in the order of the
    //! SingleThreadedCPU backend, without atomics (gennmi_runner_set_ordered); LIBRARY kernels only
    bool orderedAccumulation = false;

    //! Steps the generated stepTime() may leave queued in the device library before they are launched
    //! (gennmi_runner_set_step_queue): Runtime::stepTime() asks for one step at a time, and a model whose runner is on the
    //! resident plan runs a whole queue in one launch.  Every pull, push and synchronisation executes the queue first, so
    //! results do not depend on it; 0 launches every step when it is asked for.
    unsigned int stepQueueLength = 256;

    //! initialize() / initializeSparse() run the reference's generic initialisation code on the host (which is what makes
    //! a model start from exactly the state the SingleThreadedCPU backend gives it).  With this switch, SPARSE connectivity
    //! built by FixedProbability, FixedProbabilityNoAutapse, FixedNumberPostWithReplacement or OneToOne and per-synapse
    //! variables initialised by Constant, Uniform, Normal, NormalClipped, Exponential or Gamma are generated on the device
    //! instead (gennmi_init_sparse_*, gennmi_init_var: counter-based Philox draws from the model's seed, one stream per
    //! array): same distributions, other numbers -- as between the reference's own CPU and GPU backends.  So are the
    //! remaining built-in connectivity snippets (FixedNumberPreWithReplacement, Conv2D with kernel-initialised weights) and
    //! the variables of DENSE and kernel matrices, and unbatched, undelayed float variables of neuron populations.
    //! Everything else is initialised on the host as before.
    bool deviceInitialisation = false;

    //! Named ranges around stepTime, updateSynapses and updateNeurons for profilers (the CUDA backend's enableNVTX,
    //! cuda/backend.h:77-78): roctx ranges through gennmi_profiler_range_push / _pop.  With a step queue the ranges bracket
    //! the noting of a step, the launches happen where the queue is flushed.
    bool profilerRanges = false;

    void updateHash(boost::uuids::detail::sha1 &hash) const
    {
        PreferencesBase::updateHash(hash);
        Utils::updateHash(deviceID, hash);
        Utils::updateHash(static_cast<int>(kernelSource), hash);
        Utils::updateHash(orderedAccumulation, hash);
        Utils::updateHash(stepQueueLength, hash);
        Utils::updateHash(deviceInitialisation, hash);
        Utils::updateHash(profilerRanges, hash);
    }
};

//! Backend state of a loaded model (Runtime::getState; PyGeNN exposes it as `_Runtime`): what the device library can say about
//! the device the model runs on.  The reference's HIP backend keeps its NCCL communicator here (hip/backend.h:150-175); this
//! backend is single-GPU.
class BACKEND_EXPORT State : public Runtime::StateBase
{
public:
    //! name, architecture and compute-unit count of the current device
    std::string getDeviceName() const;
    //! device memory still free, in bytes
    size_t getFreeDeviceMemBytes() const;
    //! runs everything the device library has noted and waits for the device; throws if a kernel raised an error flag
    void synchronize() const;
};

class BACKEND_EXPORT Backend : public BackendBase
{
public:
    //! `generatedKernels`: the step's kernels are generated from the model's code (see Preferences::kernelSource);
    //! `customUpdateKernels`: the step runs on the device library's kernels and the model's custom updates on generated ones
    Backend(const Preferences &preferences, bool generatedKernels = false, bool customUpdateKernels = false);

    bool areKernelsGenerated() const { return m_GeneratedKernels; }
    //! some of the runner's modules hold device code: the Makefile builds a gfx950 code object from each of them beside the host object
    bool hasDeviceModules() const { return m_GeneratedKernels || m_CustomUpdateKernels; }

    //--------------------------------------------------------------------------
    // BackendBase virtuals
    //--------------------------------------------------------------------------
    virtual void genNeuronUpdate(CodeStream &os, FileStreamCreator streamCreator, ModelSpecMerged &modelMerged,
                                 BackendBase::MemorySpaces &memorySpaces, HostHandler preambleHandler) const final;
    virtual void genSynapseUpdate(CodeStream &os, FileStreamCreator streamCreator, ModelSpecMerged &modelMerged,
                                  BackendBase::MemorySpaces &memorySpaces, HostHandler preambleHandler) const final;
    virtual void genCustomUpdate(CodeStream &os, FileStreamCreator streamCreator, ModelSpecMerged &modelMerged,
                                 BackendBase::MemorySpaces &memorySpaces, HostHandler preambleHandler) const final;
    virtual void genInit(CodeStream &os, FileStreamCreator streamCreator, ModelSpecMerged &modelMerged,
                         BackendBase::MemorySpaces &memorySpaces, HostHandler preambleHandler) const final;

    virtual size_t getSynapticMatrixRowStride(const SynapseGroupInternal &sg) const final;

    virtual void genDefinitionsPreamble(CodeStream &os, const ModelSpecMerged &modelMerged) const final;
    virtual void genRunnerPreamble(CodeStream &os, const ModelSpecMerged &modelMerged) const final;
    virtual void genAllocateMemPreamble(CodeStream &os, const ModelSpecMerged &modelMerged) const final;
    //! backendBase.h:345-349, cuda/backend.cc:741-752
    virtual void genPushProfilerRange(CodeStream &os, const std::string &name) const final;
    virtual void genPopProfilerRange(CodeStream &os) const final;
    virtual void genFreeMemPreamble(CodeStream &os, const ModelSpecMerged &modelMerged) const final;
    virtual void genStepTimeFinalisePreamble(CodeStream &os, const ModelSpecMerged &modelMerged) const final;

    virtual std::unique_ptr<GeNN::Runtime::StateBase> createState(const Runtime::Runtime &runtime) const final;
    virtual std::unique_ptr<Runtime::ArrayBase> createArray(const Type::ResolvedType &type, size_t count,
                                                            VarLocation location, bool uninitialized) const final;
    virtual std::unique_ptr<Runtime::ArrayBase> createPopulationRNG(size_t count) const final;

    virtual void genLazyVariableDynamicAllocation(CodeStream &os, const Type::ResolvedType &type, const std::string &name,
                                                  VarLocation loc, const std::string &countVarName) const final;
    virtual void genLazyVariableDynamicPush(CodeStream &os, const Type::ResolvedType &type, const std::string &name,
                                            VarLocation loc, const std::string &countVarName) const final;
    virtual void genLazyVariableDynamicPull(CodeStream &os, const Type::ResolvedType &type, const std::string &name,
                                            VarLocation loc, const std::string &countVarName) const final;
    virtual void genMergedDynamicVariablePush(CodeStream &os, const std::string &suffix, size_t mergedGroupIdx,
                                              const std::string &groupIdx, const std::string &fieldName,
                                              const std::string &egpName) const final;

    virtual void genPopVariableInit(EnvironmentExternalBase &env, HandlerEnv handler) const final;
    virtual void genVariableInit(EnvironmentExternalBase &env, const std::string &count, const std::string &indexVarName,
                                 HandlerEnv handler) const final;
    virtual void genSparseSynapseVariableRowInit(EnvironmentExternalBase &env, HandlerEnv handler) const final;
    virtual void genDenseSynapseVariableRowInit(EnvironmentExternalBase &env, HandlerEnv handler) const final;
    virtual void genKernelSynapseVariableInit(EnvironmentExternalBase &env, SynapseInitGroupMerged &sg, HandlerEnv handler) const final;
    virtual void genKernelCustomUpdateVariableInit(EnvironmentExternalBase &env, CustomWUUpdateInitGroupMerged &cu, HandlerEnv handler) const final;

    virtual std::string getAtomicOperation(const std::string &lhsPointer, const std::string &rhsValue,
                                           const Type::ResolvedType &type, AtomicOperation op = AtomicOperation::ADD) const final;
    virtual std::string getRestrictKeyword() const final { return " __restrict__"; }

    virtual void genGlobalDeviceRNG(CodeStream &definitions, CodeStream &runner, CodeStream &allocations, CodeStream &free) const final;
    virtual void genTimer(CodeStream &definitions, CodeStream &runner, CodeStream &allocations, CodeStream &free,
                          CodeStream &stepTimeFinalise, const std::string &name, bool updateInStepTime) const final;
    virtual void genReturnFreeDeviceMemoryBytes(CodeStream &os) const final;
    virtual void genAssert(CodeStream &os, const std::string &condition) const final;

    virtual bool shouldUseNMakeBuildSystem() const final { return false; }
    virtual void genMakefilePreamble(std::ostream &os) const final;
    virtual void genMakefileLinkRule(std::ostream &os) const final;
    virtual void genMakefileCompileRule(std::ostream &os) const final;
    virtual void genNMakefilePreamble(std::ostream &os) const final;
    virtual void genNMakefileLinkRule(std::ostream &os) const final;
    virtual void genNMakefileCompileRule(std::ostream &os) const final;
    virtual void genMSBuildConfigProperties(std::ostream &os) const final;
    virtual void genMSBuildImportProps(std::ostream &os) const final;
    virtual void genMSBuildItemDefinitions(std::ostream &os) const final;
    virtual void genMSBuildCompileModule(const std::string &moduleName, std::ostream &os) const final;
    virtual void genMSBuildImportTarget(std::ostream &os) const final;

    //! Merged groups are given host pointers (see the header comment); generated code maps them to device addresses
    virtual bool isArrayDeviceObjectRequired() const final { return false; }
    virtual bool isArrayHostObjectRequired() const final { return false; }
    virtual bool isGlobalHostRNGRequired(const ModelSpecInternal &model) const final;
    virtual bool isGlobalDeviceRNGRequired(const ModelSpecInternal &model) const final { return false; }
    virtual bool isPopulationRNGInitialisedOnDevice() const final { return false; }
    //! learnPost walks columns through colLength / remap (built by gennmi_build_remap in initializeSparse())
    virtual bool isPostsynapticRemapRequired() const final { return true; }
    virtual bool isHostReductionRequired() const final { return false; }
    virtual size_t getDeviceMemoryBytes() const final;
    virtual MemorySpaces getMergedGroupMemorySpaces(const ModelSpecMerged &modelMerged) const final { return {}; }
    virtual boost::uuids::detail::sha1::digest_type getHashDigest() const final;

private:
    // generated.cc: kernels printed from the model's own code into this backend's skeletons
    void genNeuronUpdateGenerated(CodeStream &os, ModelSpecMerged &modelMerged, BackendBase::MemorySpaces &memorySpaces, HostHandler preambleHandler) const;
    void genSynapseUpdateGenerated(CodeStream &os, ModelSpecMerged &modelMerged, BackendBase::MemorySpaces &memorySpaces, HostHandler preambleHandler) const;
    void genCustomUpdateGenerated(CodeStream &os, ModelSpecMerged &modelMerged, BackendBase::MemorySpaces &memorySpaces, HostHandler preambleHandler) const;

    //! the timer of the runner's program (gennmi_program_get_time) that accumulates the launches of an update kind
    int timerId(const std::string &name) const;

    const bool m_GeneratedKernels;
    const bool m_CustomUpdateKernels;
    mutable std::map<std::string, int> m_TimerIds;
    //! neuron variables of the merged init group being printed that a device generator fills (their host loops are left out)
    mutable std::set<std::string> m_DeviceInitialisedVars;
};
}   // namespace GeNN::CodeGenerator::MI355X
