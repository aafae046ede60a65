// GeNN::CodeGenerator::MI355X::Backend — generated kernels.
//
// For models whose snippets the device library does not implement, the step's device code is generated: the model's own
// code strings — sim / threshold / reset code, postsynaptic and current-source code, weight-update code with its pre and
// post variables — are printed by GeNN's environments and pretty-printer (the transpiler stays in libgenn:
// NeuronUpdateGroupMerged::generateNeuronUpdate, PresynapticUpdateGroupMerged::generateSpikeUpdate, ...) into the
// skeletons emitted here, and the resulting translation unit is compiled for gfx950 with hipcc as part of the runner.
//
// Skeletons (what the reference's SIMT backends generate in src/genn/genn/code_generator/backendSIMT.cc:405-803, designed
// anew for 64-wide wavefronts):
//   neuron update        one lane per neuron; the model's code sets a flag where the reference appends to a shared-memory
//                        list; the flags are compacted in ascending neuron index by wave ballot, LDS scan and a tagged
//                        look-back across work-groups (include/genn_mi355x_kernel_support.h), once per population, and
//                        every spike queue of the population is written from the same positions; the ballot is the
//                        recording bitfield.  No spike-queue reset kernel: the population's last work-group stores the count.
//   presynaptic update   (spike, 64-synapse chunk of its row) items dealt round-robin to the wavefronts of a group's
//                        work-groups: a lane owns one synapse, loads of ind and the synapse variables are coalesced, a long
//                        row is shared by many wavefronts.  addToPost / addToPostDelay / addToPre are fp32 atomics.
//   postsynaptic update  (postsynaptic spike, 64-entry chunk of its column) items through the column view (remap).
//   dendritic delay      one thread per group advances the ring pointer.
// Merged-group structs are GeNN's own (same fields, same push functions); a device copy of every struct array, with host
// pointers replaced by the device buffers registered behind them, is uploaded before the first step and again whenever a
// dynamic field is pushed.  Initialisation is unchanged (the reference's generic host code, then an upload).
#include "backend.h"

#include <algorithm>
#include <set>
#include <sstream>
#include <stdexcept>

#include "code_generator/codeStream.h"
#include "code_generator/modelSpecMerged.h"
#include "code_generator/standardLibrary.h"

using namespace GeNN;
using namespace GeNN::CodeGenerator;

namespace
{
[[noreturn]] void notGenerated(const std::string &what)
{
    throw std::runtime_error("MI355X backend: generated kernels do not cover " + what);
}

// block table of one kernel: {group, first id, block in group, blocks in group} per work-group, merged groups back to back
struct BlockTable
{
    std::ostringstream entries;
    size_t numBlocks = 0;
    void add(size_t group, size_t firstId, size_t blockInGroup, size_t blocksInGroup)
    {
        entries << "{" << group << "u, " << firstId << "u, " << blockInGroup << "u, " << blocksInGroup << "u}, ";
        if((++numBlocks % 4) == 0) { entries << std::endl; }
    }
};

// device copy of a merged group's struct array: declaration, and the statements that translate and upload it
template<typename G>
void genDeviceStructArray(CodeStream &decl, CodeStream &upload, const BackendBase &backend, const G &g, const std::string &name)
{
    const std::string type = "Merged" + name + "Group" + std::to_string(g.getIndex());
    const std::string host = "merged" + name + "Group" + std::to_string(g.getIndex());
    const std::string dev = "d_" + host;
    const size_t count = g.getGroups().size();
    decl << "static " << type << " *" << dev << " = nullptr;" << std::endl;
    upload << "// " << host << std::endl;
    {
        CodeStream::Scope b(upload);
        upload << "static " << type << " staging[" << count << "];" << std::endl;
        upload << "for(unsigned int g = 0; g < " << count << "; g++)";
        {
            CodeStream::Scope b2(upload);
            upload << "staging[g] = " << host << "[g];" << std::endl;
            for(const auto &f : g.getSortedFields(backend)) {
                if(f.type.isPointer()) {
                    upload << "staging[g]." << f.name << " = gennmiDev(staging[g]." << f.name << ");" << std::endl;
                }
            }
        }
        upload << "if(!" << dev << ") { void *p = nullptr; GENNMI_CHECK(gennmi_malloc(&p, sizeof(staging))); " << dev << " = (" << type << "*)p; }" << std::endl;
        upload << "GENNMI_CHECK(gennmi_memcpy_to_device(" << dev << ", staging, sizeof(staging)));" << std::endl;
    }
}
// gennrand_* as the reference's backends declare them (cuda/backend.cc:35-43), over gennmi_kernel::Rng.  The draws have fp32
// resolution whatever the model's precision (a double-precision model gets them converted).
EnvironmentLibrary::Library simRNGLibrary(const Type::ResolvedType &scalar)
{
    const std::string cast = (scalar == Type::Float) ? "" : ("(" + scalar.getName() + ")");
    return {
        {"gennrand", {Type::ResolvedType::createFunction(Type::Uint32, {}), "gennmi_kernel::rngWord($(_rng))"}},
        {"gennrand_uniform", {Type::ResolvedType::createFunction(scalar, {}), cast + "gennmi_kernel::rngUniform($(_rng))"}},
        {"gennrand_normal", {Type::ResolvedType::createFunction(scalar, {}), cast + "gennmi_kernel::rngNormal($(_rng))"}},
        {"gennrand_exponential", {Type::ResolvedType::createFunction(scalar, {}), cast + "gennmi_kernel::rngExponential($(_rng))"}},
        {"gennrand_log_normal", {Type::ResolvedType::createFunction(scalar, {scalar, scalar}), cast + "gennmi_kernel::rngLogNormal($(_rng), (float)($(0)), (float)($(1)))"}},
        {"gennrand_gamma", {Type::ResolvedType::createFunction(scalar, {scalar}), cast + "gennmi_kernel::rngGamma($(_rng), (float)($(0)))"}},
        {"gennrand_binomial", {Type::ResolvedType::createFunction(Type::Uint32, {Type::Uint32, scalar}), "gennmi_kernel::rngBinomial($(_rng), $(0), (float)($(1)))"}},
    };
}
}   // anonymous namespace

namespace GeNN::CodeGenerator::MI355X
{
//--------------------------------------------------------------------------
void Backend::genNeuronUpdateGenerated(CodeStream &os, ModelSpecMerged &modelMerged, BackendBase::MemorySpaces &memorySpaces,
                                       HostHandler preambleHandler) const
{
    const ModelSpecInternal &model = modelMerged.getModel();
    // batches: the grid's second dimension (backendCUDAHIP.cc:332-338 does the same); every batch compacts its own queue
    const unsigned int batchSize = model.getBatchSize();
    const std::string timeType = model.getTimePrecision().getName();
    const EnvironmentLibrary::Library simRNGFunctions = simRNGLibrary(model.getPrecision());
    const bool recording = model.isRecordingInUse();

    std::ostringstream kernelStream, declStream, uploadStream, argStream, paramStream;
    CodeStream kernel(kernelStream), decl(declStream), upload(uploadStream);
    BlockTable table;

    EnvironmentLibrary kernelEnv(kernel, StandardLibrary::getMathsFunctions());
    bool anyRNG = false;
    size_t maxEventGroups = 0;      // spike-like event conditions of one population: each compacts a queue of its own
    {   // (environments write what they hold when they go out of scope: the kernel's text is complete after this block)
    // gennrand_* of simulation code: words of a counter-based generator, see gennmi_kernel::Rng (`_rng` exists in the
    // populations that need it)
    EnvironmentLibrary rngEnv(kernelEnv, simRNGFunctions);
    EnvironmentExternal funcEnv(rngEnv);
    funcEnv.add(model.getTimePrecision().addConst(), "t", "t");
    funcEnv.add(Type::Uint32.addConst(), "batch", (batchSize > 1) ? "blockIdx.y" : "0");
    funcEnv.add(model.getTimePrecision().addConst(), "dt", Type::writeNumeric(model.getDT(), model.getTimePrecision()));

    modelMerged.genMergedNeuronUpdateGroups(
        *this, memorySpaces,
        [&](auto &n)
        {
            const auto &arch = n.getArchetype();
            maxEventGroups = std::max(maxEventGroups, n.getMergedSpikeEventGroups().size());

            const size_t firstBlock = table.numBlocks;
            for(size_t g = 0; g < n.getGroups().size(); g++) {
                const size_t num = n.getGroups()[g].get().getNumNeurons();
                const size_t blocks = (num + 255) / 256;
                for(size_t b = 0; b < blocks; b++) { table.add(g, b * 256, b, blocks); }
            }
            const std::string structArray = "mergedNeuronUpdateGroup" + std::to_string(n.getIndex());
            argStream << ", d_" << structArray;
            paramStream << ", const MergedNeuronUpdateGroup" << n.getIndex() << " *" << structArray;

            funcEnv.getStream() << "// merged neuron update group " << n.getIndex() << std::endl;
            funcEnv.getStream() << (firstBlock == 0 ? "if" : "else if") << "(blockIdx.x < " << table.numBlocks << "u)";
            CodeStream::Scope b(funcEnv.getStream());
            funcEnv.getStream() << "const gennmi_kernel::BlockEntry entry = gennmiNeuronBlocks[blockIdx.x];" << std::endl;
            funcEnv.getStream() << "const auto *group = &" << structArray << "[entry.group];" << std::endl;
            funcEnv.getStream() << "const unsigned int id = entry.firstId + threadIdx.x;" << std::endl;
            funcEnv.getStream() << "bool gennmiSpiked = false;" << std::endl;
            for(const auto &e : n.getMergedSpikeEventGroups()) { funcEnv.getStream() << "bool gennmiEvent" << e.getIndex() << " = false;" << std::endl; }

            EnvironmentGroupMergedField<NeuronUpdateGroupMerged> groupEnv(funcEnv, n);
            buildStandardEnvironment(groupEnv, batchSize);
            groupEnv.add(Type::Uint32.addConst(), "id", "id");
            // where a batch's entries of a per-neuron array (spike queue, spike times) begin
            // (with axonal delay: in the slot of the population's ring that this step writes, the one *spk_que_ptr names after
            // the queue-update kernel has advanced it; GeNN's generic code copies delayed variables of neurons that did not
            // spike from the slot read to the slot written, neuronUpdateGroupMerged.cc:714-770)
            const std::string queueOffset = n.getWriteVarIndex(arch.isSpikeDelayRequired(), batchSize, VarAccessDim::BATCH | VarAccessDim::ELEMENT, "");
            const std::string countIndex = arch.isSpikeDelayRequired() ? ((batchSize > 1) ? "$(_write_batch_delay_slot)" : "$(_write_delay_slot)") : "$(batch)";
            if(arch.isSimRNGRequired()) {
                // one generator stream per population: 2000 + its place in the model's name-ordered list of populations
                anyRNG = true;
                groupEnv.addField(Type::Uint32.addConst(), "_rng_stream", Type::Uint32, "rngStream",
                                  [&model](const NeuronGroupInternal &g, size_t)
                                  {
                                      return Type::NumericValue((uint64_t)(2000 + std::distance(model.getNeuronGroups().cbegin(), model.getNeuronGroups().find(g.getName()))));
                                  });
                groupEnv.add(Type::Uint32, "_rng", "gennmiRng",
                             {groupEnv.addInitialiser("gennmi_kernel::Rng gennmiRng = gennmi_kernel::rngBegin(gennmiSeed, $(_rng_stream), "
                                                      + n.getVarIndex(batchSize, VarAccessDim::BATCH | VarAccessDim::ELEMENT, "$(id)") + ", gennmiStep);")});
            }
            if(arch.isSpikeRecordingEnabled()) {
                groupEnv.printLine("const unsigned int numRecordingWords = ($(num_neurons) + 31) / 32;");
            }
            groupEnv.print("if($(id) < $(num_neurons))");
            {
                CodeStream::Scope b2(groupEnv.getStream());
                n.generateNeuronUpdate(
                    groupEnv, batchSize,
                    // a true spike: weight-update pre / post spike code, spike time; the queue is written after the
                    // population's flags have been compacted (below), the recording word comes from the ballot
                    [&n, &arch, &queueOffset, batchSize](EnvironmentExternalBase &env)
                    {
                        n.generateWUVarUpdate(env, batchSize);
                        if(arch.isSpikeTimeRequired()) { env.printLine("$(_st)[" + queueOffset + "$(id)] = $(t);"); }
                        env.getStream() << "gennmiSpiked = true;" << std::endl;
                    },
                    // a spike-like event of one of the population's conditions: flagged here, queued below like the true spikes
                    [](EnvironmentExternalBase &env, NeuronUpdateGroupMerged::SynSpikeEvent &e)
                    {
                        env.getStream() << "gennmiEvent" << e.getIndex() << " = true;" << std::endl;
                    });
            }
            groupEnv.printLine("const gennmi_kernel::QueueSlot slot = gennmi_kernel::orderedSlot(gennmiSpiked, entry.blockInGroup, entry.blocksInGroup, "
                               "blockIdx.x - entry.blockInGroup, gennmiAgg + (size_t)2 * gridDim.x * blockIdx.y, gennmiAgg + (size_t)2 * gridDim.x * blockIdx.y + gridDim.x, "
                               "gennmiTag, gennmiError);");
            if(arch.isSpikeRecordingEnabled()) {
                groupEnv.printLine("gennmi_kernel::recordBallot(&$(_record_spk)[((size_t)recordingTimestep * " + std::to_string(batchSize) + "u + $(batch)) * numRecordingWords], "
                                   "$(id), $(id) < $(num_neurons), slot.ballot);");
            }
            // spike-like events: one ordered compaction per condition (its own look-back words), the ballot as recording bitfield
            if(!n.getMergedSpikeEventGroups().empty()) {
                const std::string eventOffset = n.getWriteVarIndex(arch.isSpikeEventDelayRequired(), batchSize, VarAccessDim::BATCH | VarAccessDim::ELEMENT, "");
                const std::string eventCountIndex = arch.isSpikeEventDelayRequired() ? ((batchSize > 1) ? "$(_write_batch_delay_slot)" : "$(_write_delay_slot)") : "$(batch)";
                const bool recordEvents = arch.isSpikeEventRecordingEnabled();
                if(recordEvents && !arch.isSpikeRecordingEnabled()) {
                    groupEnv.printLine("const unsigned int numRecordingWords = ($(num_neurons) + 31) / 32;");
                }
                n.generateSpikeEvents(
                    groupEnv,
                    [&eventOffset, &eventCountIndex, &arch, recordEvents, batchSize](EnvironmentExternalBase &env, NeuronUpdateGroupMerged::SynSpikeEvent &e)
                    {
                        const std::string k = std::to_string(e.getIndex());
                        const std::string region = "gennmiAgg + (size_t)2 * gridDim.x * (gridDim.y * " + std::to_string(e.getIndex() + 1) + "u + blockIdx.y)";
                        env.printLine("const gennmi_kernel::QueueSlot eventSlot" + k + " = gennmi_kernel::orderedSlot(gennmiEvent" + k + ", entry.blockInGroup, entry.blocksInGroup, "
                                      "blockIdx.x - entry.blockInGroup, " + region + ", " + region + " + gridDim.x, gennmiTag, gennmiError);");
                        if(recordEvents) {
                            env.printLine("gennmi_kernel::recordBallot(&$(_record_spk_event)[((size_t)recordingTimestep * " + std::to_string(batchSize) + "u + $(batch)) * numRecordingWords], "
                                          "$(id), $(id) < $(num_neurons), eventSlot" + k + ".ballot);");
                        }
                        if(arch.isSpikeEventTimeRequired()) { env.printLine("if(gennmiEvent" + k + ") { $(_set)[" + eventOffset + "$(id)] = $(t); }"); }
                        env.print("if(eventSlot" + k + ".ok)");
                        CodeStream::Scope b3(env.getStream());
                        env.printLine("if(gennmiEvent" + k + ") { $(_spk_event)[" + eventOffset + "eventSlot" + k + ".position] = $(id); }");
                        env.printLine("if(eventSlot" + k + ".writeTotal) { $(_spk_cnt_event)[" + eventCountIndex + "] = eventSlot" + k + ".total; }");
                    });
            }
            // every spike queue of the population (one per fused outgoing / incoming spike target) from the same positions
            n.generateSpikes(
                groupEnv,
                [&queueOffset, &countIndex](EnvironmentExternalBase &env)
                {
                    env.print("if(slot.ok)");
                    CodeStream::Scope b3(env.getStream());
                    env.printLine("if(gennmiSpiked) { $(_spk)[" + queueOffset + "slot.position] = $(id); }");
                    env.printLine("if(slot.writeTotal) { $(_spk_cnt)[" + countIndex + "] = slot.total; }");
                });
        });
    }

    // Previous spike (and event) times: every neuron in last step's queue gets prev_st = t - dt, in a kernel that runs before
    // the ring pointers move on (backendSIMT.cc:320-368, 1897-1925)
    std::ostringstream prevStream, prevArgs, prevParams;
    BlockTable prevTable;
    if(!modelMerged.getMergedNeuronPrevSpikeTimeUpdateGroups().empty()) {
        CodeStream prev(prevStream);
        EnvironmentLibrary prevLib(prev, StandardLibrary::getMathsFunctions());
        EnvironmentExternal prevEnv(prevLib);
        prevEnv.add(model.getTimePrecision().addConst(), "t", "t");
        prevEnv.add(Type::Uint32.addConst(), "batch", (batchSize > 1) ? "blockIdx.y" : "0");
        prevEnv.add(model.getTimePrecision().addConst(), "dt", Type::writeNumeric(model.getDT(), model.getTimePrecision()));
        modelMerged.genMergedNeuronPrevSpikeTimeUpdateGroups(
            *this, memorySpaces,
            [&](auto &n)
            {
                const auto &arch = n.getArchetype();
                const size_t firstBlock = prevTable.numBlocks;
                for(size_t g = 0; g < n.getGroups().size(); g++) {
                    const size_t blocks = (n.getGroups()[g].get().getNumNeurons() + 255) / 256;
                    for(size_t b = 0; b < blocks; b++) { prevTable.add(g, b * 256, b, blocks); }
                }
                const std::string structArray = "mergedNeuronPrevSpikeTimeUpdateGroup" + std::to_string(n.getIndex());
                prevArgs << ", d_" << structArray;
                prevParams << ", const MergedNeuronPrevSpikeTimeUpdateGroup" << n.getIndex() << " *" << structArray;
                prevEnv.getStream() << (firstBlock == 0 ? "if" : "else if") << "(blockIdx.x < " << prevTable.numBlocks << "u)";
                CodeStream::Scope b(prevEnv.getStream());
                prevEnv.getStream() << "const gennmi_kernel::BlockEntry entry = gennmiPrevSpikeTimeBlocks[blockIdx.x];" << std::endl;
                prevEnv.getStream() << "const auto *group = &" << structArray << "[entry.group];" << std::endl;
                prevEnv.getStream() << "const unsigned int id = entry.firstId + threadIdx.x;" << std::endl;
                EnvironmentGroupMergedField<NeuronPrevSpikeTimeUpdateGroupMerged> groupEnv(prevEnv, n);
                buildStandardEnvironment(groupEnv, batchSize);
                groupEnv.add(Type::Uint32.addConst(), "id", "id");
                if(arch.isDelayRequired()) {
                    groupEnv.printLine("const unsigned int lastSlot = *$(_spk_que_ptr)" + ((batchSize > 1) ? " + ($(batch) * " + std::to_string(arch.getNumDelaySlots()) + "u)" : std::string("")) + ";");
                    groupEnv.printLine("const unsigned int lastOffset = lastSlot * $(num_neurons);");
                }
                auto stamp = [&arch, batchSize](EnvironmentExternalBase &env, bool trueSpike)
                {
                    const std::string suffix = trueSpike ? "" : "_event", time = trueSpike ? "st" : "set";
                    if(trueSpike ? arch.isSpikeDelayRequired() : arch.isSpikeEventDelayRequired()) {
                        env.printLine("if($(id) < $(_spk_cnt" + suffix + ")[lastSlot]) { $(_prev_" + time + ")[lastOffset + $(_spk" + suffix + ")[lastOffset + $(id)]] = $(t) - $(dt); }");
                    }
                    else {
                        const std::string offset = (batchSize > 1) ? "$(_batch_offset) + " : "";
                        env.printLine("if($(id) < $(_spk_cnt" + suffix + ")[$(batch)]) { $(_prev_" + time + ")[" + offset + "$(_spk" + suffix + ")[" + offset + "$(id)]] = $(t) - $(dt); }");
                    }
                };
                if(arch.isPrevSpikeTimeRequired()) { n.generateSpikes(groupEnv, [&stamp](EnvironmentExternalBase &env) { stamp(env, true); }); }
                if(arch.isPrevSpikeEventTimeRequired()) { n.generateSpikeEvents(groupEnv, [&stamp](EnvironmentExternalBase &env) { stamp(env, false); }); }
            });
    }
    const bool anyPrevTimes = prevTable.numBlocks > 0;

    // Populations with delay slots: their ring pointer moves on before the update (backendSIMT.cc:372-401; one thread per group).
    // Without delay slots that kernel would only clear counts that the compaction overwrites anyway, and is left out.
    const bool anyDelaySlots = std::any_of(model.getNeuronGroups().cbegin(), model.getNeuronGroups().cend(),
                                           [](const auto &n) { return n.second.isDelayRequired(); });
    std::ostringstream queueStream, queueArgs, queueParams;
    if(anyDelaySlots) {
        CodeStream queue(queueStream);
        EnvironmentLibrary queueLib(queue, StandardLibrary::getMathsFunctions());
        EnvironmentExternal queueEnv(queueLib);
        modelMerged.genMergedNeuronSpikeQueueUpdateGroups(
            *this, memorySpaces,
            [&](auto &n)
            {
                const std::string structArray = "mergedNeuronSpikeQueueUpdateGroup" + std::to_string(n.getIndex());
                queueArgs << (queueArgs.str().empty() ? "" : ", ") << "d_" << structArray;
                queueParams << (queueParams.str().empty() ? "" : ", ") << "MergedNeuronSpikeQueueUpdateGroup" << n.getIndex() << " *" << structArray;
                queueEnv.getStream() << "for(unsigned int g = threadIdx.x; g < " << n.getGroups().size() << "u; g += blockDim.x)";
                CodeStream::Scope b(queueEnv.getStream());
                queueEnv.getStream() << "auto *group = &" << structArray << "[g];" << std::endl;
                EnvironmentGroupMergedField<NeuronSpikeQueueUpdateGroupMerged> groupEnv(queueEnv, n);
                buildStandardEnvironment(groupEnv, batchSize);
                n.genSpikeQueueUpdate(groupEnv, batchSize);
            });
    }

    // struct definitions, host arrays and their push functions are GeNN's own
    modelMerged.genMergedNeuronUpdateGroupStructs(os, *this);
    modelMerged.genMergedNeuronUpdateGroupHostStructArrayPush(os, *this);
    if(anyDelaySlots) {
        modelMerged.genMergedNeuronSpikeQueueUpdateStructs(os, *this);
        modelMerged.genMergedNeuronSpikeQueueUpdateHostStructArrayPush(os, *this);
    }
    if(anyPrevTimes) {
        modelMerged.genMergedNeuronPrevSpikeTimeUpdateStructs(os, *this);
        modelMerged.genMergedNeuronPrevSpikeTimeUpdateHostStructArrayPush(os, *this);
    }
    preambleHandler(os);
    for(const auto &n : modelMerged.getMergedNeuronUpdateGroups()) {
        genDeviceStructArray(decl, upload, *this, n, "NeuronUpdate");
    }
    if(anyDelaySlots) {
        for(const auto &n : modelMerged.getMergedNeuronSpikeQueueUpdateGroups()) { genDeviceStructArray(decl, upload, *this, n, "NeuronSpikeQueueUpdate"); }
    }
    if(anyPrevTimes) {
        for(const auto &n : modelMerged.getMergedNeuronPrevSpikeTimeUpdateGroups()) { genDeviceStructArray(decl, upload, *this, n, "NeuronPrevSpikeTimeUpdate"); }
    }

    os << declStream.str();
    os << "static unsigned long long *gennmiNeuronAgg = nullptr;" << std::endl;
    os << "static uint32_t *gennmiNeuronError = nullptr;" << std::endl;
    os << "static unsigned int gennmiNeuronLaunches = 0;" << std::endl;
    os << "__device__ const gennmi_kernel::BlockEntry gennmiNeuronBlocks[] = {" << std::endl << table.entries.str() << "{0u, 0u, 0u, 0u}};" << std::endl;
    os << std::endl;
    os << "void gennmiUploadNeuronGroups()";
    {
        CodeStream::Scope b(os);
        os << uploadStream.str();
        os << "if(!gennmiNeuronAgg)";
        {
            CodeStream::Scope b2(os);
            os << "void *p = nullptr;" << std::endl;
            os << "GENNMI_CHECK(gennmi_malloc(&p, " << 2 * std::max<size_t>(1, table.numBlocks) * batchSize * (1 + maxEventGroups) << " * sizeof(unsigned long long)));" << std::endl;
            os << "GENNMI_CHECK(gennmi_memset(p, 0, " << 2 * std::max<size_t>(1, table.numBlocks) * batchSize * (1 + maxEventGroups) << " * sizeof(unsigned long long)));" << std::endl;
            os << "gennmiNeuronAgg = (unsigned long long*)p;" << std::endl;
            os << "GENNMI_CHECK(gennmi_malloc(&p, sizeof(uint32_t)));" << std::endl;
            os << "GENNMI_CHECK(gennmi_memset(p, 0, sizeof(uint32_t)));" << std::endl;
            os << "gennmiNeuronError = (uint32_t*)p;" << std::endl;
        }
    }
    os << std::endl;
    if(anyPrevTimes) {
        os << "__device__ const gennmi_kernel::BlockEntry gennmiPrevSpikeTimeBlocks[] = {" << std::endl << prevTable.entries.str() << "{0u, 0u, 0u, 0u}};" << std::endl;
        os << "__global__ __launch_bounds__(256) void gennmiPrevSpikeTimeKernel(" << timeType << " t" << prevParams.str() << ")";
        CodeStream::Scope b(os);
        os << prevStream.str();
    }
    if(anyDelaySlots) {
        os << "__global__ void gennmiSpikeQueueUpdateKernel(" << queueParams.str() << ")";
        CodeStream::Scope b(os);
        os << queueStream.str();
    }
    os << std::endl;
    os << "__global__ __launch_bounds__(256) void gennmiNeuronUpdateKernel(" << timeType << " t, unsigned int recordingTimestep, uint32_t gennmiTag, "
          "unsigned long long *gennmiAgg, uint32_t *gennmiError, unsigned long long gennmiSeed, unsigned long long gennmiStep" << paramStream.str() << ")";
    {
        CodeStream::Scope b(os);
        os << kernelStream.str();
    }
    os << std::endl;
    os << "void updateNeurons(" << model.getTimePrecision().getName() << " t";
    if(recording) { os << ", unsigned int recordingTimestep"; }
    os << ")";
    {
        CodeStream::Scope b(os);
        os << "gennmiEnsureFinalised();" << std::endl;
        if(anyPrevTimes) { os << "gennmiPrevSpikeTimeKernel<<<dim3(" << prevTable.numBlocks << ", " << batchSize << "), dim3(256), 0, 0>>>(t" << prevArgs.str() << ");" << std::endl; }
        if(anyDelaySlots) { os << "gennmiSpikeQueueUpdateKernel<<<dim3(1), dim3(64), 0, 0>>>(" << queueArgs.str() << ");" << std::endl; }
        const bool timing = model.isTimingEnabled();
        if(timing) { os << "hipEventRecord(neuronUpdateStart, 0);" << std::endl; }
        if(table.numBlocks > 0) {
            // the tag of a launch: differs from one launch to the next, never 0 (the look-back words start out zero)
            os << "gennmiNeuronLaunches = (gennmiNeuronLaunches == 0xFFFFFFFFu) ? 1u : gennmiNeuronLaunches + 1u;" << std::endl;
            // (the generator's step counter: calls of updateNeurons so far; the seed: the model's, or one drawn at load time)
            os << "static unsigned long long gennmiNeuronStep = 0;" << std::endl;
            os << "gennmiNeuronUpdateKernel<<<dim3(" << table.numBlocks << ", " << batchSize << "), dim3(256), 0, 0>>>(t, " << (recording ? "recordingTimestep" : "0u")
               << ", gennmiNeuronLaunches, gennmiNeuronAgg, gennmiNeuronError, "
               << (anyRNG ? ((model.getSeed() != 0) ? (std::to_string(model.getSeed()) + "ull") : std::string("gennmiRandomSeed()")) : std::string("0ull"))
               << ", gennmiNeuronStep++" << argStream.str() << ");" << std::endl;
            os << "if(hipGetLastError() != hipSuccess) { throw std::runtime_error(\"updateNeurons: kernel launch failed\"); }" << std::endl;
        }
        if(timing) { os << "hipEventRecord(neuronUpdateStop, 0);" << std::endl; }
    }
    os << std::endl;
    // bounded waits of the compaction that expired are reported where the reference's backends check for launch errors
    os << "void gennmiCheckNeuronKernels()";
    {
        CodeStream::Scope b(os);
        os << "if(!gennmiNeuronError) { return; }" << std::endl;
        os << "uint32_t flag = 0;" << std::endl;
        os << "GENNMI_CHECK(gennmi_memcpy_from_device(&flag, gennmiNeuronError, sizeof(flag)));" << std::endl;
        os << "if(flag) { throw std::runtime_error(\"updateNeurons: a work-group's bounded wait for spike-queue offsets expired\"); }" << std::endl;
    }
}
//--------------------------------------------------------------------------
void Backend::genSynapseUpdateGenerated(CodeStream &os, ModelSpecMerged &modelMerged, BackendBase::MemorySpaces &memorySpaces,
                                        HostHandler preambleHandler) const
{
    const ModelSpecInternal &model = modelMerged.getModel();
    const double dt = model.getDT();
    const unsigned int batchSize = model.getBatchSize();

    const std::string timeType = model.getTimePrecision().getName();
    const EnvironmentLibrary::Library simRNGFunctions = simRNGLibrary(model.getPrecision());

    std::ostringstream declStream, uploadStream;
    CodeStream decl(declStream), upload(uploadStream);

    // every kernel's body, arguments and block table
    struct KernelText
    {
        std::ostringstream body, args, params;
        BlockTable table;
    };
    KernelText delay, dynamics, pre, post;
    auto makeEnv = [&model, &simRNGFunctions](CodeStream &stream, EnvironmentLibrary &lib, auto use)
    {
        EnvironmentLibrary rngLib(lib, simRNGFunctions);        // (gennrand_* of weight-update code: `_rng` exists where it is used)
        EnvironmentExternal funcEnv(rngLib);
        funcEnv.add(model.getTimePrecision().addConst(), "t", "t");
        funcEnv.add(Type::Uint32.addConst(), "batch", (model.getBatchSize() > 1) ? "blockIdx.y" : "0");
        funcEnv.add(model.getTimePrecision().addConst(), "dt", Type::writeNumeric(model.getDT(), model.getTimePrecision()));
        (void)stream;
        use(funcEnv);
    };

    // Random numbers in weight-update code: a generator per synapse and step — counter (synapse id of the batch, step, call),
    // stream 3000 + 8 x the projection's place in the model's name-ordered list + the kind of code (0 spike, 1 spike-like
    // event, 2 postsynaptic spike, 3 synapse dynamics, 4 postsynaptic spike-like event), key = the model's seed.  (The reference skips ahead in one Philox
    // sequence per thread, backendCUDAHIP.cc:497, so there as here no two backends draw the same numbers.)
    bool anySynapseRNG = false;
    auto addSynapseRng = [&model, &anySynapseRNG, batchSize](auto &codeEnv, const SynapseGroupInternal &, const auto &tokens, unsigned int kind)
    {
        if(!Utils::isRNGRequired(tokens)) { return; }
        anySynapseRNG = true;
        const std::string k = std::to_string(kind);
        codeEnv.addField(Type::Uint32.addConst(), "_rng_stream" + k, Type::Uint32, "rngStream" + k,
                         [&model, kind](const SynapseGroupInternal &g, size_t)
                         {
                             return Type::NumericValue((uint64_t)(3000 + 8 * std::distance(model.getSynapseGroups().cbegin(), model.getSynapseGroups().find(g.getName())) + kind));
                         });
        const std::string element = (batchSize > 1) ? "(unsigned long long)$(_syn_batch_offset) + $(id_syn)" : "(unsigned long long)$(id_syn)";
        codeEnv.add(Type::Uint32, "_rng", "gennmiRng",
                    {codeEnv.addInitialiser("gennmi_kernel::Rng gennmiRng = gennmi_kernel::rngBegin(gennmiSeed, $(_rng_stream" + k + "), " + element + ", gennmiStep);")});
    };

    // ---- synapse dynamics: every (padded) synapse every step, a grid-stride walk per group (backendSIMT.cc:805-863 gives each
    // synapse a thread)
    {
        CodeStream stream(dynamics.body);
        EnvironmentLibrary lib(stream, StandardLibrary::getMathsFunctions());
        makeEnv(stream, lib, [&](EnvironmentExternal &funcEnv)
        {
            modelMerged.genMergedSynapseDynamicsGroups(
                *this, memorySpaces,
                [&](auto &s)
                {
                    const auto &arch = s.getArchetype();
                    const auto matrix = arch.getMatrixType();
                    const bool sparse = (matrix & SynapseMatrixConnectivity::SPARSE);
                    const bool dense = (matrix & SynapseMatrixConnectivity::DENSE) && (matrix & SynapseMatrixWeight::INDIVIDUAL);
                    if(!sparse && !dense) { notGenerated("connectivity other than SPARSE and DENSE (projection '" + arch.getName() + "')"); }
                    const size_t firstBlock = dynamics.table.numBlocks;
                    for(size_t g = 0; g < s.getGroups().size(); g++) {
                        const auto &sg = s.getGroups()[g].get();
                        const size_t rowLen = sparse ? getSynapticMatrixRowStride(sg) : sg.getTrgNeuronGroup()->getNumNeurons();
                        const size_t blocks = std::clamp<size_t>((sg.getSrcNeuronGroup()->getNumNeurons() * rowLen + 255) / 256, 1, 1024);
                        for(size_t b = 0; b < blocks; b++) { dynamics.table.add(g, 0, b, blocks); }
                    }
                    const std::string structArray = "mergedSynapseDynamicsGroup" + std::to_string(s.getIndex());
                    dynamics.args << ", d_" << structArray;
                    dynamics.params << ", const MergedSynapseDynamicsGroup" << s.getIndex() << " *" << structArray;

                    funcEnv.getStream() << "// merged synapse dynamics group " << s.getIndex() << std::endl;
                    funcEnv.getStream() << (firstBlock == 0 ? "if" : "else if") << "(blockIdx.x < " << dynamics.table.numBlocks << "u)";
                    CodeStream::Scope b(funcEnv.getStream());
                    funcEnv.getStream() << "const gennmi_kernel::BlockEntry entry = gennmiSynapseDynamicsBlocks[blockIdx.x];" << std::endl;
                    funcEnv.getStream() << "const auto *group = &" << structArray << "[entry.group];" << std::endl;
                    EnvironmentGroupMergedField<SynapseDynamicsGroupMerged> groupEnv(funcEnv, s);
                    buildStandardEnvironment(groupEnv, batchSize);
                    const auto indexType = getSynapseIndexType(s);
                    const std::string indexTypeName = indexType.getName();
                    groupEnv.printLine(std::string("const unsigned int rowSpan = ") + (sparse ? "$(_row_stride)" : "$(num_post)") + ";");
                    groupEnv.printLine("const unsigned long long numSynapses = (unsigned long long)$(num_pre) * rowSpan;");
                    groupEnv.getStream() << "for(unsigned long long item = (unsigned long long)entry.blockInGroup * 256u + threadIdx.x; item < numSynapses; "
                                            "item += (unsigned long long)entry.blocksInGroup * 256u)";
                    {
                        CodeStream::Scope b2(groupEnv.getStream());
                        EnvironmentGroupMergedField<SynapseDynamicsGroupMerged> synEnv(groupEnv, s);
                        synEnv.getStream() << "const unsigned int row = (unsigned int)(item / rowSpan);" << std::endl;
                        synEnv.getStream() << "const unsigned int col = (unsigned int)(item % rowSpan);" << std::endl;
                        if(sparse) {
                            synEnv.print("if(col < $(_row_length)[row])");
                        }
                        {
                            CodeStream::Scope b3(synEnv.getStream());
                            EnvironmentGroupMergedField<SynapseDynamicsGroupMerged> codeEnv(synEnv, s);
                            codeEnv.add(Type::Uint32.addConst(), "id_pre", "row");
                            codeEnv.add(indexType.addConst(), "id_syn", "idSyn",
                                        {codeEnv.addInitialiser("const " + indexTypeName + " idSyn = (" + indexTypeName + ")item;")});
                            if(sparse) {
                                codeEnv.add(Type::Uint32.addConst(), "id_post", "idPost",
                                            {codeEnv.addInitialiser("const unsigned int idPost = $(_ind)[item];")});
                            }
                            else {
                                codeEnv.add(Type::Uint32.addConst(), "id_post", "col");
                            }
                            codeEnv.add(Type::getAddToPrePostDelay(s.getScalarType()), "addToPostDelay",
                                        "gennmi_kernel::addScalar(&$(_den_delay)[" + s.getPostDenDelayIndex(batchSize, "$(id_post)", "$(1)") + "], $(0))");
                            codeEnv.add(Type::getAddToPrePost(s.getScalarType()), "addToPost",
                                        "gennmi_kernel::addScalar(&$(_out_post)[" + s.getPostISynIndex(batchSize, "$(id_post)") + "], $(0))");
                            codeEnv.add(Type::getAddToPrePost(s.getScalarType()), "addToPre",
                                        "gennmi_kernel::addScalar(&$(_out_pre)[" + s.getPreISynIndex(batchSize, "$(id_pre)") + "], $(0))");
                            addSynapseRng(codeEnv, arch, arch.getWUInitialiser().getSynapseDynamicsCodeTokens(), 3);
                            s.generateSynapseUpdate(*this, codeEnv, batchSize, dt);
                        }
                    }
                });
        });
    }

    // ---- dendritic delay pointers: one thread per group
    {
        CodeStream stream(delay.body);
        EnvironmentLibrary lib(stream, StandardLibrary::getMathsFunctions());
        makeEnv(stream, lib, [&](EnvironmentExternal &funcEnv)
        {
            modelMerged.genMergedSynapseDendriticDelayUpdateGroups(
                *this, memorySpaces,
                [&](auto &sg)
                {
                    const std::string structArray = "mergedSynapseDendriticDelayUpdateGroup" + std::to_string(sg.getIndex());
                    delay.table.numBlocks++;
                    delay.args << ", d_" << structArray;
                    delay.params << ", const MergedSynapseDendriticDelayUpdateGroup" << sg.getIndex() << " *" << structArray;
                    funcEnv.getStream() << "for(unsigned int g = threadIdx.x; g < " << sg.getGroups().size() << "u; g += blockDim.x)";
                    CodeStream::Scope b(funcEnv.getStream());
                    funcEnv.getStream() << "const auto *group = &" << structArray << "[g];" << std::endl;
                    EnvironmentGroupMergedField<SynapseDendriticDelayUpdateGroupMerged> groupEnv(funcEnv, sg);
                    buildStandardEnvironment(groupEnv, 1);
                    sg.generateSynapseUpdate(groupEnv);
                });
        });
    }

    // ---- presynaptic update
    {
        CodeStream stream(pre.body);
        EnvironmentLibrary lib(stream, StandardLibrary::getMathsFunctions());
        makeEnv(stream, lib, [&](EnvironmentExternal &funcEnv)
        {
            modelMerged.genMergedPresynapticUpdateGroups(
                *this, memorySpaces,
                [&](auto &s)
                {
                    const auto &arch = s.getArchetype();
                    const auto matrix = arch.getMatrixType();
                    const bool sparse = (matrix & SynapseMatrixConnectivity::SPARSE);
                    const bool dense = (matrix & SynapseMatrixConnectivity::DENSE);
                    const bool toeplitz = (matrix & SynapseMatrixConnectivity::TOEPLITZ);
                    const bool bitmask = (matrix & SynapseMatrixConnectivity::BITMASK);
                    const bool procedural = (matrix & SynapseMatrixConnectivity::PROCEDURAL);
                    if(!sparse && !dense && !toeplitz && !bitmask && !procedural) { notGenerated("this matrix type (projection '" + arch.getName() + "')"); }
                    if((matrix & SynapseMatrixWeight::PROCEDURAL) && !procedural && !dense) {
                        notGenerated("weights regenerated from their initialisation snippet on connectivity other than DENSE and PROCEDURAL (projection '" + arch.getName() + "')");
                    }
                    if(!arch.isPreSpikeRequired() && !arch.isPreSpikeEventRequired()) { return; }
                    // PROCEDURAL: a row is the connectivity snippet's row build code, run by `threadsPerSpike` lanes that share the
                    // target range between them (SynapseGroup::setNumThreadsPerSpike)
                    const size_t threadsPerSpike = procedural ? arch.getNumThreadsPerSpike() : 1;

                    const size_t firstBlock = pre.table.numBlocks;
                    for(size_t g = 0; g < s.getGroups().size(); g++) {
                        const auto &sg = s.getGroups()[g].get();
                        const size_t rowLen = procedural ? threadsPerSpike : (sparse || toeplitz || bitmask) ? getSynapticMatrixRowStride(sg) : sg.getTrgNeuronGroup()->getNumNeurons();
                        const size_t chunks = (rowLen + 63) / 64;
                        // enough wavefronts for ~1.5 % of the source population firing in one step, at most 128 work-groups
                        const size_t blocks = std::clamp<size_t>((sg.getSrcNeuronGroup()->getNumNeurons() * chunks + 255) / 256, 1, 128);
                        for(size_t b = 0; b < blocks; b++) { pre.table.add(g, 0, b, blocks); }
                    }
                    const std::string structArray = "mergedPresynapticUpdateGroup" + std::to_string(s.getIndex());
                    pre.args << ", d_" << structArray;
                    pre.params << ", const MergedPresynapticUpdateGroup" << s.getIndex() << " *" << structArray;

                    funcEnv.getStream() << "// merged presynaptic update group " << s.getIndex() << std::endl;
                    funcEnv.getStream() << (firstBlock == 0 ? "if" : "else if") << "(blockIdx.x < " << pre.table.numBlocks << "u)";
                    CodeStream::Scope b(funcEnv.getStream());
                    funcEnv.getStream() << "const gennmi_kernel::BlockEntry entry = gennmiPresynapticBlocks[blockIdx.x];" << std::endl;
                    funcEnv.getStream() << "const auto *group = &" << structArray << "[entry.group];" << std::endl;
                    EnvironmentGroupMergedField<PresynapticUpdateGroupMerged> groupEnv(funcEnv, s);
                    buildStandardEnvironment(groupEnv, batchSize);
                    groupEnv.printLine(std::string("const unsigned int rowSpan = ") + (procedural ? (std::to_string(threadsPerSpike) + "u") : (sparse || toeplitz || bitmask) ? "$(_row_stride)" : "$(num_post)") + ";");
                    groupEnv.getStream() << "const unsigned int chunksPerRow = (rowSpan + 63u) / 64u;" << std::endl;
                    groupEnv.getStream() << "const unsigned int numWaves = entry.blocksInGroup * 4u;" << std::endl;
                    // the queue of spike-like events first, then the true spikes (the reference's order, backendSIMT.cc:745-760);
                    // either is a walk over (entry of the queue, 64-synapse chunk of its row) items
                    auto walk = [&](bool trueSpike)
                    {
                        const std::string suffix = trueSpike ? "" : "_event";
                        const auto *src = arch.getSrcNeuronGroup();
                        // (axonal delay: the slot of the source's ring written `delay` steps ago, presynapticUpdateStrategySIMT.cc:224-247)
                        const bool preDelay = src->isDelayRequired() && (trueSpike ? src->isSpikeQueueRequired() : src->isSpikeEventQueueRequired());
                        CodeStream::Scope b1(groupEnv.getStream());
                        groupEnv.printLine("const unsigned int numSpikes = $(_src_spk_cnt" + suffix + ")[" + s.getPreSlot(preDelay, batchSize) + "];");
                        groupEnv.getStream() << "const unsigned long long numItems = (unsigned long long)numSpikes * chunksPerRow;" << std::endl;
                        groupEnv.getStream() << "for(unsigned long long item = entry.blockInGroup * 4u + (threadIdx.x / 64u); item < numItems; item += numWaves)";
                        CodeStream::Scope b2(groupEnv.getStream());
                        EnvironmentGroupMergedField<PresynapticUpdateGroupMerged> synEnv(groupEnv, s);
                        synEnv.getStream() << "const unsigned int spike = (unsigned int)(item / chunksPerRow);" << std::endl;
                        synEnv.getStream() << "const unsigned int j = (unsigned int)(item % chunksPerRow) * 64u + (threadIdx.x & 63u);" << std::endl;
                        synEnv.printLine("const unsigned int idPre = $(_src_spk" + suffix + ")[" + s.getPreVarIndex(preDelay, batchSize, VarAccessDim::BATCH | VarAccessDim::ELEMENT, "spike") + "];");
                        synEnv.add(Type::Uint32.addConst(), "id_pre", "idPre");
                        if(procedural) {
                            // A row of a PROCEDURAL matrix is the connectivity snippet's row build code, run afresh for every spike:
                            // lane j of an item takes the j-th share of the target range, and the snippet's addSynapse(idPost,
                            // kernel indices...) becomes the weight-update code (presynapticUpdateStrategySIMT.cc:425-565).  Random
                            // numbers of the row build code and of weights regenerated from their initialisation snippet come from
                            // one counter-based generator per (row, lane): key = the model's seed, stream 2k + 1 for the k-th
                            // projection by name, counter = the lane's number, step 0 — so a row is the same every time it is built
                            // (the reference skips ahead in one Philox sequence to the same end).
                            EnvironmentGroupMergedField<PresynapticUpdateGroupMerged> rowEnv(synEnv, s);
                            const std::string tps = std::to_string(threadsPerSpike);
                            // (the population's size under another name: `num_post` itself becomes a lane's share below)
                            rowEnv.add(Type::Uint32.addConst(), "_num_post", "$(num_post)");
                            if(Utils::isRNGRequired(arch.getSparseConnectivityInitialiser().getRowBuildCodeTokens())
                               || ((matrix & SynapseMatrixWeight::PROCEDURAL) && Utils::isRNGRequired(arch.getWUInitialiser().getVarInitialisers())))
                            {
                                anySynapseRNG = true;
                                rowEnv.addField(Type::Uint32.addConst(), "_rng_stream_row", Type::Uint32, "rngStreamRow",
                                                [&model](const SynapseGroupInternal &g, size_t)
                                                {
                                                    return Type::NumericValue((uint64_t)(2 * std::distance(model.getSynapseGroups().cbegin(), model.getSynapseGroups().find(g.getName())) + 1));
                                                });
                                rowEnv.add(Type::Uint32, "_rng", "gennmiRng",
                                           {rowEnv.addInitialiser("gennmi_kernel::Rng gennmiRng = gennmi_kernel::rngBegin(gennmiSeed, $(_rng_stream_row), (unsigned long long)idPre * " + tps + "u + j, 0ull);")});
                            }
                            std::ostringstream updateStream;
                            CodeStream update(updateStream);
                            {
                                CodeStream::Scope bu(update);
                                EnvironmentExternal updateEnv(rowEnv, update);
                                updateEnv.add(Type::Uint32.addConst(), "id_post", "idPost", {updateEnv.addInitialiser("const unsigned int idPost = $(0);")});
                                for(size_t i = 0; i < arch.getKernelSize().size(); i++) {
                                    const std::string iStr = std::to_string(i);
                                    updateEnv.add(Type::Uint32.addConst(), "id_kernel_" + iStr, "idKernel" + iStr,
                                                  {updateEnv.addInitialiser("const unsigned int idKernel" + iStr + " = $(" + std::to_string(i + 1) + ");")});
                                }
                                updateEnv.add(Type::getAddToPrePostDelay(s.getScalarType()), "addToPostDelay",
                                              "gennmi_kernel::addScalar(&$(_den_delay)[" + s.getPostDenDelayIndex(batchSize, "$(id_post)", "$(1)") + "], $(0))");
                                updateEnv.add(Type::getAddToPrePost(s.getScalarType()), "addToPost",
                                              "gennmi_kernel::addScalar(&$(_out_post)[" + s.getPostISynIndex(batchSize, "$(id_post)") + "], $(0))");
                                updateEnv.add(Type::getAddToPrePost(s.getScalarType()), "addToPre",
                                              "gennmi_kernel::addScalar(&$(_out_pre)[" + s.getPreISynIndex(batchSize, "$(id_pre)") + "], $(0))");
                                if(trueSpike) { s.generateSpikeUpdate(*this, updateEnv, batchSize, dt); }
                                else { s.generateSpikeEventUpdate(*this, updateEnv, batchSize, dt); }
                            }
                            rowEnv.getStream() << "if(j < " << tps << "u)";
                            CodeStream::Scope bt(rowEnv.getStream());
                            EnvironmentExternal connEnv(rowEnv);
                            connEnv.add(Type::Uint32.addConst(), "num_threads", tps);
                            connEnv.add(Type::Uint32.addConst(), "id_thread", "j");
                            if(threadsPerSpike > 1) {
                                const size_t perThread = connEnv.addInitialiser("const unsigned int numPostPerThread = ($(_num_post) + " + tps + "u - 1u) / " + tps + "u;");
                                connEnv.add(Type::Uint32.addConst(), "id_post_begin", "idPostBegin",
                                            {perThread, connEnv.addInitialiser("const unsigned int idPostBegin = j * numPostPerThread;")});
                                // (the last lanes' shares end with the population)
                                connEnv.add(Type::Uint32.addConst(), "num_post", "numPostOfThread",
                                            {perThread, connEnv.addInitialiser("const unsigned int numPostOfThread = (j * numPostPerThread >= $(_num_post)) ? 0u : min(numPostPerThread, $(_num_post) - j * numPostPerThread);")});
                            }
                            else {
                                connEnv.add(Type::Uint32.addConst(), "id_post_begin", "0");
                            }
                            const auto addSynapseType = Type::ResolvedType::createFunction(
                                Type::Void, std::vector<Type::ResolvedType>{1ull + arch.getKernelSize().size(), Type::Uint32});
                            connEnv.add(addSynapseType, "addSynapse", updateStream.str());
                            s.generateProceduralConnectivity(connEnv);
                            return;
                        }
                        if(toeplitz) {
                            // A row of a Toeplitz matrix is the connectivity snippet's diagonal build code run for (presynaptic
                            // neuron, diagonal): lane j of an item takes diagonal j, and the snippet's addSynapse(idPost, kernel
                            // indices...) becomes the weight-update code with those values (presynapticUpdateStrategySIMT.cc:784-917)
                            std::ostringstream updateStream;
                            CodeStream update(updateStream);
                            {
                                CodeStream::Scope bu(update);
                                EnvironmentExternal updateEnv(synEnv, update);
                                updateEnv.add(Type::Uint32.addConst(), "id_post", "idPost", {updateEnv.addInitialiser("const unsigned int idPost = $(0);")});
                                for(size_t i = 0; i < arch.getKernelSize().size(); i++) {
                                    const std::string iStr = std::to_string(i);
                                    updateEnv.add(Type::Uint32.addConst(), "id_kernel_" + iStr, "idKernel" + iStr,
                                                  {updateEnv.addInitialiser("const unsigned int idKernel" + iStr + " = $(" + std::to_string(i + 1) + ");")});
                                }
                                updateEnv.add(Type::getAddToPrePostDelay(s.getScalarType()), "addToPostDelay",
                                              "gennmi_kernel::addScalar(&$(_den_delay)[" + s.getPostDenDelayIndex(batchSize, "$(id_post)", "$(1)") + "], $(0))");
                                updateEnv.add(Type::getAddToPrePost(s.getScalarType()), "addToPost",
                                              "gennmi_kernel::addScalar(&$(_out_post)[" + s.getPostISynIndex(batchSize, "$(id_post)") + "], $(0))");
                                updateEnv.add(Type::getAddToPrePost(s.getScalarType()), "addToPre",
                                              "gennmi_kernel::addScalar(&$(_out_pre)[" + s.getPreISynIndex(batchSize, "$(id_pre)") + "], $(0))");
                                if(trueSpike) { s.generateSpikeUpdate(*this, updateEnv, batchSize, dt); }
                                else { s.generateSpikeEventUpdate(*this, updateEnv, batchSize, dt); }
                            }
                            synEnv.print("if(j < $(_row_stride))");
                            CodeStream::Scope bt(synEnv.getStream());
                            EnvironmentExternal diagEnv(synEnv);
                            diagEnv.add(Type::Uint32.addConst(), "id_diag", "j");
                            const auto addSynapseType = Type::ResolvedType::createFunction(
                                Type::Void, std::vector<Type::ResolvedType>{1ull + arch.getKernelSize().size(), Type::Uint32});
                            s.generateToeplitzConnectivity(
                                diagEnv,
                                [addSynapseType](auto &env, auto &errorHandler)
                                {
                                    env.define(Transpiler::Token{Transpiler::Token::Type::IDENTIFIER, "addSynapse", 0}, addSynapseType, errorHandler);
                                    env.define(Transpiler::Token{Transpiler::Token::Type::IDENTIFIER, "id_pre", 0}, Type::Uint32.addConst(), errorHandler);
                                },
                                [addSynapseType, &updateStream](auto &env, auto generateBody)
                                {
                                    EnvironmentExternal bodyEnv(env);
                                    bodyEnv.add(addSynapseType, "addSynapse", updateStream.str());
                                    generateBody(bodyEnv);
                                });
                            return;
                        }
                        const auto indexType = getSynapseIndexType(s);
                        const std::string indexTypeName = indexType.getName();
                        if(sparse) {
                            synEnv.print("if(j < $(_row_length)[idPre])");
                        }
                        else if(bitmask) {
                            // a bit per (source, target), rows padded to whole words, most significant bit of a word first
                            // (presynapticUpdateStrategySIMT.cc:276-281)
                            synEnv.getStream() << "const " << indexTypeName << " bit = ((" << indexTypeName << ")idPre * rowSpan) + j;" << std::endl;
                            synEnv.print("if(j < $(num_post) && ($(_gp)[bit / 32] & (0x80000000u >> (bit & 31))))");
                        }
                        else {
                            synEnv.print("if(j < $(num_post))");
                        }
                        CodeStream::Scope b3(synEnv.getStream());
                        EnvironmentGroupMergedField<PresynapticUpdateGroupMerged> codeEnv(synEnv, s);
                        if(sparse) {
                            codeEnv.add(indexType.addConst(), "id_syn", "idSyn",
                                        {codeEnv.addInitialiser("const " + indexTypeName + " idSyn = ((" + indexTypeName + ")idPre * $(_row_stride)) + j;")});
                            codeEnv.add(Type::Uint32.addConst(), "id_post", "idPost",
                                        {codeEnv.addInitialiser("const unsigned int idPost = $(_ind)[$(id_syn)];")});
                        }
                        else {
                            codeEnv.add(Type::Uint32.addConst(), "id_post", "j");
                            codeEnv.add(indexType.addConst(), "id_syn", "idSyn",
                                        {codeEnv.addInitialiser("const " + indexTypeName + " idSyn = ((" + indexTypeName + ")idPre * " + (bitmask ? "rowSpan" : "$(num_post)") + ") + j;")});
                        }
                        // (DENSE with weights regenerated from their initialisation snippet at every event: GeNN allows such snippets no
                        // random numbers — synapseGroup.cc — so the snippet's code is evaluated as it stands, generateSpikeUpdate does it)
                        codeEnv.add(Type::getAddToPrePostDelay(s.getScalarType()), "addToPostDelay",
                                    "gennmi_kernel::addScalar(&$(_den_delay)[" + s.getPostDenDelayIndex(batchSize, "$(id_post)", "$(1)") + "], $(0))");
                        codeEnv.add(Type::getAddToPrePost(s.getScalarType()), "addToPost",
                                    "gennmi_kernel::addScalar(&$(_out_post)[" + s.getPostISynIndex(batchSize, "$(id_post)") + "], $(0))");
                        codeEnv.add(Type::getAddToPrePost(s.getScalarType()), "addToPre",
                                    "gennmi_kernel::addScalar(&$(_out_pre)[" + s.getPreISynIndex(batchSize, "$(id_pre)") + "], $(0))");
                        if(trueSpike) {
                            addSynapseRng(codeEnv, arch, arch.getWUInitialiser().getPreSpikeSynCodeTokens(), 0);
                            s.generateSpikeUpdate(*this, codeEnv, batchSize, dt);
                        }
                        else {
                            addSynapseRng(codeEnv, arch, arch.getWUInitialiser().getPreEventSynCodeTokens(), 1);
                            s.generateSpikeEventUpdate(*this, codeEnv, batchSize, dt);
                        }
                    };
                    if(arch.isPreSpikeEventRequired()) { walk(false); }
                    if(arch.isPreSpikeRequired()) { walk(true); }
                });
        });
    }

    // ---- postsynaptic update (learnPost) through the column view
    {
        CodeStream stream(post.body);
        EnvironmentLibrary lib(stream, StandardLibrary::getMathsFunctions());
        makeEnv(stream, lib, [&](EnvironmentExternal &funcEnv)
        {
            modelMerged.genMergedPostsynapticUpdateGroups(
                *this, memorySpaces,
                [&](auto &s)
                {
                    const auto &arch = s.getArchetype();
                    const auto matrix = arch.getMatrixType();
                    const bool sparse = (matrix & SynapseMatrixConnectivity::SPARSE);
                    const bool dense = (matrix & SynapseMatrixConnectivity::DENSE) && (matrix & SynapseMatrixWeight::INDIVIDUAL);
                    if(!sparse && !dense) { notGenerated("connectivity other than SPARSE and DENSE (projection '" + arch.getName() + "')"); }
                    if(!arch.isPostSpikeRequired() && !arch.isPostSpikeEventRequired()) { return; }

                    const size_t firstBlock = post.table.numBlocks;
                    for(size_t g = 0; g < s.getGroups().size(); g++) {
                        const auto &sg = s.getGroups()[g].get();
                        const size_t colLen = sparse ? sg.getMaxSourceConnections() : sg.getSrcNeuronGroup()->getNumNeurons();
                        const size_t chunks = (colLen + 63) / 64;
                        const size_t blocks = std::clamp<size_t>((sg.getTrgNeuronGroup()->getNumNeurons() * chunks + 255) / 256, 1, 128);
                        for(size_t b = 0; b < blocks; b++) { post.table.add(g, 0, b, blocks); }
                    }
                    const std::string structArray = "mergedPostsynapticUpdateGroup" + std::to_string(s.getIndex());
                    post.args << ", d_" << structArray;
                    post.params << ", const MergedPostsynapticUpdateGroup" << s.getIndex() << " *" << structArray;

                    funcEnv.getStream() << "// merged postsynaptic update group " << s.getIndex() << std::endl;
                    funcEnv.getStream() << (firstBlock == 0 ? "if" : "else if") << "(blockIdx.x < " << post.table.numBlocks << "u)";
                    CodeStream::Scope b(funcEnv.getStream());
                    funcEnv.getStream() << "const gennmi_kernel::BlockEntry entry = gennmiPostsynapticBlocks[blockIdx.x];" << std::endl;
                    funcEnv.getStream() << "const auto *group = &" << structArray << "[entry.group];" << std::endl;
                    EnvironmentGroupMergedField<PostsynapticUpdateGroupMerged> groupEnv(funcEnv, s);
                    buildStandardEnvironment(groupEnv, batchSize);
                    groupEnv.printLine(std::string("const unsigned int colSpan = ") + (sparse ? "$(_col_stride)" : "$(num_pre)") + ";");
                    groupEnv.getStream() << "const unsigned int chunksPerCol = (colSpan + 63u) / 64u;" << std::endl;
                    groupEnv.getStream() << "const unsigned int numWaves = entry.blocksInGroup * 4u;" << std::endl;
                    // the queue of postsynaptic spike-like events first, then the true spikes (single_threaded_cpu/backend.cc:573-580)
                    auto walk = [&](bool trueSpike)
                    {
                    const std::string suffix = trueSpike ? "" : "_event";
                    const auto *trg = arch.getTrgNeuronGroup();
                    // (back-propagation delay: the slot of the target's ring written `delay` steps ago, backendSIMT.cc:1822-1835)
                    const bool postDelay = trg->isDelayRequired() && (trueSpike ? trg->isSpikeQueueRequired() : trg->isSpikeEventQueueRequired());
                    CodeStream::Scope b1(groupEnv.getStream());
                    groupEnv.printLine("const unsigned int numSpikes = $(_trg_spk_cnt" + suffix + ")[" + s.getPostSlot(postDelay, batchSize) + "];");
                    groupEnv.getStream() << "const unsigned long long numItems = (unsigned long long)numSpikes * chunksPerCol;" << std::endl;
                    // (items are dealt to the work-groups first, then to their wavefronts: a column walk is a stream of scattered accesses,
                    // which a compute unit issues at about one lane per clock, so the first items should each find a compute unit of their own)
                    groupEnv.getStream() << "for(unsigned long long item = (threadIdx.x / 64u) * entry.blocksInGroup + entry.blockInGroup; item < numItems; item += numWaves)";
                    {
                        CodeStream::Scope b2(groupEnv.getStream());
                        EnvironmentGroupMergedField<PostsynapticUpdateGroupMerged> synEnv(groupEnv, s);
                        synEnv.printLine("const unsigned int spike = $(_trg_spk" + suffix + ")[" + s.getPostVarIndex(postDelay, batchSize, VarAccessDim::BATCH | VarAccessDim::ELEMENT, "(unsigned int)(item / chunksPerCol)") + "];");
                        synEnv.getStream() << "const unsigned int i = (unsigned int)(item % chunksPerCol) * 64u + (threadIdx.x & 63u);" << std::endl;
                        if(sparse) {
                            synEnv.print("if(i < $(_col_length)[spike])");
                        }
                        else {
                            synEnv.print("if(i < $(num_pre))");
                        }
                        {
                            CodeStream::Scope b3(synEnv.getStream());
                            EnvironmentGroupMergedField<PostsynapticUpdateGroupMerged> codeEnv(synEnv, s);
                            if(sparse) {
                                const size_t colMajor = codeEnv.addInitialiser("const unsigned int colMajorIndex = (spike * $(_col_stride)) + i;");
                                const size_t rowMajor = codeEnv.addInitialiser("const unsigned int rowMajorIndex = $(_remap)[colMajorIndex];");
                                const size_t idPre = codeEnv.addInitialiser("const unsigned int idPre = rowMajorIndex / $(_row_stride);");
                                codeEnv.add(Type::Uint32.addConst(), "id_pre", "idPre", {colMajor, rowMajor, idPre});
                                codeEnv.add(Type::Uint32.addConst(), "id_syn", "rowMajorIndex", {colMajor, rowMajor});
                            }
                            else {
                                codeEnv.add(Type::Uint32.addConst(), "id_pre", "i");
                                codeEnv.add(Type::Uint32.addConst(), "id_syn", "idSyn",
                                            {codeEnv.addInitialiser("const unsigned int idSyn = (i * $(num_post)) + spike;")});
                            }
                            codeEnv.add(Type::Uint32.addConst(), "id_post", "spike");
                            codeEnv.add(Type::getAddToPrePost(s.getScalarType()), "addToPre",
                                        "gennmi_kernel::addScalar(&$(_out_pre)[" + s.getPreISynIndex(batchSize, "$(id_pre)") + "], $(0))");
                            if(trueSpike) {
                                addSynapseRng(codeEnv, arch, arch.getWUInitialiser().getPostSpikeSynCodeTokens(), 2);
                                s.generateSpikeUpdate(*this, codeEnv, batchSize, dt);
                            }
                            else {
                                addSynapseRng(codeEnv, arch, arch.getWUInitialiser().getPostEventSynCodeTokens(), 4);
                                s.generateSpikeEventUpdate(*this, codeEnv, batchSize, dt);
                            }
                        }
                    }
                    };
                    if(arch.isPostSpikeEventRequired()) { walk(false); }
                    if(arch.isPostSpikeRequired()) { walk(true); }
                });
        });
    }

    // struct definitions, host arrays and push functions (GeNN's own), then the device copies
    modelMerged.genMergedSynapseDendriticDelayUpdateStructs(os, *this);
    modelMerged.genMergedPresynapticUpdateGroupStructs(os, *this);
    modelMerged.genMergedPostsynapticUpdateGroupStructs(os, *this);
    modelMerged.genMergedSynapseDynamicsGroupStructs(os, *this);
    modelMerged.genMergedSynapseDendriticDelayUpdateHostStructArrayPush(os, *this);
    modelMerged.genMergedPresynapticUpdateGroupHostStructArrayPush(os, *this);
    modelMerged.genMergedPostsynapticUpdateGroupHostStructArrayPush(os, *this);
    modelMerged.genMergedSynapseDynamicsGroupHostStructArrayPush(os, *this);
    preambleHandler(os);
    for(const auto &g : modelMerged.getMergedSynapseDendriticDelayUpdateGroups()) { genDeviceStructArray(decl, upload, *this, g, "SynapseDendriticDelayUpdate"); }
    for(const auto &g : modelMerged.getMergedPresynapticUpdateGroups()) { genDeviceStructArray(decl, upload, *this, g, "PresynapticUpdate"); }
    for(const auto &g : modelMerged.getMergedPostsynapticUpdateGroups()) { genDeviceStructArray(decl, upload, *this, g, "PostsynapticUpdate"); }
    for(const auto &g : modelMerged.getMergedSynapseDynamicsGroups()) { genDeviceStructArray(decl, upload, *this, g, "SynapseDynamics"); }

    os << declStream.str();
    os << "__device__ const gennmi_kernel::BlockEntry gennmiPresynapticBlocks[] = {" << std::endl << pre.table.entries.str() << "{0u, 0u, 0u, 0u}};" << std::endl;
    os << "__device__ const gennmi_kernel::BlockEntry gennmiPostsynapticBlocks[] = {" << std::endl << post.table.entries.str() << "{0u, 0u, 0u, 0u}};" << std::endl;
    os << "__device__ const gennmi_kernel::BlockEntry gennmiSynapseDynamicsBlocks[] = {" << std::endl << dynamics.table.entries.str() << "{0u, 0u, 0u, 0u}};" << std::endl;
    os << std::endl;
    os << "void gennmiUploadSynapseGroups()";
    {
        CodeStream::Scope b(os);
        os << uploadStream.str();
    }
    os << std::endl;
    const bool anyDelay = delay.table.numBlocks > 0, anyPre = pre.table.numBlocks > 0, anyPost = post.table.numBlocks > 0, anyDynamics = dynamics.table.numBlocks > 0;
    if(anyDynamics) {
        os << "__global__ __launch_bounds__(256) void gennmiSynapseDynamicsKernel(" << timeType << " t, unsigned long long gennmiSeed, unsigned long long gennmiStep" << dynamics.params.str() << ")";
        CodeStream::Scope b(os);
        os << dynamics.body.str();
    }
    if(anyDelay) {
        os << "__global__ void gennmiDendriticDelayUpdateKernel(" << timeType << " t" << delay.params.str() << ")";
        CodeStream::Scope b(os);
        os << delay.body.str();
    }
    if(anyPre) {
        os << "__global__ __launch_bounds__(256) void gennmiPresynapticUpdateKernel(" << timeType << " t, unsigned long long gennmiSeed, unsigned long long gennmiStep" << pre.params.str() << ")";
        CodeStream::Scope b(os);
        os << pre.body.str();
    }
    if(anyPost) {
        os << "__global__ __launch_bounds__(256) void gennmiPostsynapticUpdateKernel(" << timeType << " t, unsigned long long gennmiSeed, unsigned long long gennmiStep" << post.params.str() << ")";
        CodeStream::Scope b(os);
        os << post.body.str();
    }
    os << std::endl;
    os << "void updateSynapses(" << model.getTimePrecision().getName() << " t)";
    {
        CodeStream::Scope b(os);
        os << "gennmiEnsureFinalised();" << std::endl;
        // order of the reference's updateSynapses (backendCUDAHIP.cc:548-589): ring pointers, synapse dynamics, presynaptic, postsynaptic
        if(anyDelay) { os << "gennmiDendriticDelayUpdateKernel<<<dim3(1), dim3(64), 0, 0>>>(t" << delay.args.str() << ");" << std::endl; }
        // (the generators' step counter: calls of updateSynapses so far; the seed: the model's, or one drawn at load time)
        const std::string seedAndStep = std::string(", ") + (anySynapseRNG ? ((model.getSeed() != 0) ? (std::to_string(model.getSeed()) + "ull") : std::string("gennmiRandomSeed()")) : std::string("0ull"))
                                        + ", gennmiSynapseStep";
        os << "static unsigned long long gennmiSynapseStep = 0;" << std::endl;
        // (timers exist for the kinds of update the model has merged groups of, generateRunner.cc:177-199)
        const bool timing = model.isTimingEnabled();
        auto timer = [&](bool exists, const char *name, const char *edge) { if(timing && exists) { os << "hipEventRecord(" << name << edge << ", 0);" << std::endl; } };
        timer(!modelMerged.getMergedSynapseDynamicsGroups().empty(), "synapseDynamics", "Start");
        if(anyDynamics) { os << "gennmiSynapseDynamicsKernel<<<dim3(" << dynamics.table.numBlocks << ", " << batchSize << "), dim3(256), 0, 0>>>(t" << seedAndStep << dynamics.args.str() << ");" << std::endl; }
        timer(!modelMerged.getMergedSynapseDynamicsGroups().empty(), "synapseDynamics", "Stop");
        timer(!modelMerged.getMergedPresynapticUpdateGroups().empty(), "presynapticUpdate", "Start");
        if(anyPre) { os << "gennmiPresynapticUpdateKernel<<<dim3(" << pre.table.numBlocks << ", " << batchSize << "), dim3(256), 0, 0>>>(t" << seedAndStep << pre.args.str() << ");" << std::endl; }
        timer(!modelMerged.getMergedPresynapticUpdateGroups().empty(), "presynapticUpdate", "Stop");
        timer(!modelMerged.getMergedPostsynapticUpdateGroups().empty(), "postsynapticUpdate", "Start");
        if(anyPost) { os << "gennmiPostsynapticUpdateKernel<<<dim3(" << post.table.numBlocks << ", " << batchSize << "), dim3(256), 0, 0>>>(t" << seedAndStep << post.args.str() << ");" << std::endl; }
        timer(!modelMerged.getMergedPostsynapticUpdateGroups().empty(), "postsynapticUpdate", "Stop");
        os << "gennmiSynapseStep++;" << std::endl;
        os << "if(hipGetLastError() != hipSuccess) { throw std::runtime_error(\"updateSynapses: kernel launch failed\"); }" << std::endl;
    }
}
//--------------------------------------------------------------------------
// Custom updates: update<Group>(timestep), one function per update-group name (Runtime::customUpdate looks them up by that
// name, runtime.cc:114-118), launching up to four kernels of the group's merged custom updates:
//   per neuron      one lane per element (the batch is the grid's second dimension); a reduction over batches loops over them
//                   in the lane that owns the element; a reduction over neurons takes one work-group per batch — lanes stride
//                   over the population, partial results meet through wave shuffles and LDS
//   per synapse     one lane per entry of the padded matrix (SPARSE: those beyond the row's length idle), of the dense matrix
//                   or of the kernel; work-groups find their group by bisection, not through a table entry each
//   transpose       64 x 64 tiles of a DENSE matrix through LDS: rows are read and written 256 bytes at a time
//   connectivity    (custom connectivity updates, which run first) a lane per row of a SPARSE matrix runs the row update code;
//                   the column views of projections that learn from postsynaptic spikes are rebuilt afterwards
// (what backendSIMT.cc:868-1270 does with 32-wide tiles and one warp per reduction).  The update code itself, its variable
// and variable-reference indexing (delay slots, batches, shared dimensions) are GeNN's: generateCustomUpdate.
//--------------------------------------------------------------------------
void Backend::genCustomUpdateGenerated(CodeStream &os, ModelSpecMerged &modelMerged, BackendBase::MemorySpaces &memorySpaces,
                                       HostHandler preambleHandler) const
{
    const ModelSpecInternal &model = modelMerged.getModel();
    const unsigned int batchSize = model.getBatchSize();
    std::set<std::string> groupNames;
    for(const auto &c : model.getCustomUpdates()) { groupNames.insert(c.second.getUpdateGroupName()); }
    for(const auto &c : model.getCustomWUUpdates()) { groupNames.insert(c.second.getUpdateGroupName()); }
    for(const auto &c : model.getCustomConnectivityUpdates()) { groupNames.insert(c.second.getUpdateGroupName()); }
    auto refuseRNG = [](const auto &arch)
    {
        if(Utils::isRNGRequired(arch.getUpdateCodeTokens())) { notGenerated("random numbers in custom update code (custom update '" + arch.getName() + "')"); }
    };

    std::ostringstream declStream, uploadStream, deviceStream, hostStream;
    CodeStream decl(declStream), upload(uploadStream), device(deviceStream), host(hostStream);
    const std::string timeType = model.getTimePrecision().getName();
    const EnvironmentLibrary::Library simRNGFunctions = simRNGLibrary(model.getPrecision());
    auto reduceOps = [this](auto &env, const std::vector<ReductionTarget> &targets)
    {
        for(const auto &r : targets) { env.printLine(getReductionOperation("_lr" + r.name, "$(" + r.name + ")", r.access, r.type) + ";"); }
    };

    // beside the device library's kernels: the arrays a custom update may have written (variable references that are not
    // read-only, the transpose target) are named to the library afterwards, which refreshes what it derives from them
    auto noteWrites = [this](std::ostringstream &notes, const auto &c, const std::string &structName, const std::vector<std::string> &extra)
    {
        if(m_GeneratedKernels) { return; }
        std::vector<std::string> written(extra);
        for(const auto &v : c.getArchetype().getModel()->getVarRefs()) {
            if(v.access != VarAccessMode::READ_ONLY) { written.push_back(v.name); }
        }
        const auto fields = c.getSortedFields(*this);
        for(const auto &w : written) {
            if(std::any_of(fields.cbegin(), fields.cend(), [&w](const auto &f) { return f.name == w; })) {
                notes << "for(unsigned int g = 0; g < " << c.getGroups().size() << "u; g++) { GENNMI_CHECK(gennmi_note_mirror_write(merged" << structName
                      << "Group" << c.getIndex() << "[g]." << w << ")); }" << std::endl;
            }
        }
    };

    for(const std::string &name : groupNames) {
        std::ostringstream notes;
        // ---- per-neuron custom updates
        std::ostringstream neuronBody, neuronArgs, neuronParams;
        BlockTable neuronTable;
        {
            CodeStream body(neuronBody);
            EnvironmentLibrary lib(body, StandardLibrary::getMathsFunctions());
            EnvironmentExternal funcEnv(lib);
            funcEnv.add(model.getTimePrecision().addConst(), "t", "t");
            funcEnv.add(model.getTimePrecision().addConst(), "dt", Type::writeNumeric(model.getDT(), model.getTimePrecision()));
            modelMerged.genMergedCustomUpdateGroups(
                *this, memorySpaces, name,
                [&](auto &c)
                {
                    const auto &arch = c.getArchetype();
                    refuseRNG(arch);
                    const bool perElement = (arch.getDims() & VarAccessDim::ELEMENT);
                    const bool batched = (arch.getDims() & VarAccessDim::BATCH) && (batchSize > 1);
                    const bool oneBlock = arch.isNeuronReduction() || !perElement;
                    const size_t firstBlock = neuronTable.numBlocks;
                    for(size_t g = 0; g < c.getGroups().size(); g++) {
                        const size_t blocks = oneBlock ? 1 : ((size_t)c.getGroups()[g].get().getNumNeurons() + 255) / 256;
                        for(size_t b = 0; b < blocks; b++) { neuronTable.add(g, b * 256, b, blocks); }
                    }
                    const std::string structArray = "mergedCustomUpdateGroup" + std::to_string(c.getIndex());
                    neuronArgs << ", d_" << structArray;
                    neuronParams << ", const MergedCustomUpdateGroup" << c.getIndex() << " *" << structArray;

                    funcEnv.getStream() << "// merged custom update group " << c.getIndex() << std::endl;
                    funcEnv.getStream() << (firstBlock == 0 ? "if" : "else if") << "(blockIdx.x < " << neuronTable.numBlocks << "u)";
                    CodeStream::Scope b(funcEnv.getStream());
                    funcEnv.getStream() << "const gennmi_kernel::BlockEntry entry = gennmiCustomUpdate" << name << "Blocks[blockIdx.x];" << std::endl;
                    funcEnv.getStream() << "const auto *group = &" << structArray << "[entry.group];" << std::endl;
                    // (updates that are not batched run in the first of the grid's batch rows only)
                    const std::string firstRowOnly = (batchSize > 1) ? "blockIdx.y == 0u && " : "";

                    EnvironmentGroupMergedField<CustomUpdateGroupMerged> groupEnv(funcEnv, c);
                    buildSizeEnvironment(groupEnv);
                    if(arch.isBatchReduction()) {
                        groupEnv.getStream() << "const unsigned int id = entry.firstId + threadIdx.x;" << std::endl;
                        groupEnv.add(Type::Uint32.addConst(), "id", "id");
                        groupEnv.print("if(" + firstRowOnly + "$(id) < $(num_neurons))");
                        CodeStream::Scope b2(groupEnv.getStream());
                        const auto targets = genInitReductionTargets(groupEnv.getStream(), c, batchSize, groupEnv["id"]);
                        groupEnv.getStream() << "for(unsigned int batch = 0; batch < " << batchSize << "u; batch++)";
                        {
                            CodeStream::Scope b3(groupEnv.getStream());
                            EnvironmentGroupMergedField<CustomUpdateGroupMerged> batchEnv(groupEnv, c);
                            batchEnv.add(Type::Uint32.addConst(), "batch", "batch");
                            buildStandardEnvironment(batchEnv, batchSize);
                            c.generateCustomUpdate(batchEnv, batchSize, [&](auto &env, const auto&) { reduceOps(env, targets); });
                        }
                        for(const auto &r : targets) { groupEnv.printLine("group->" + r.name + "[" + r.index + "] = _lr" + r.name + ";"); }
                    }
                    else if(arch.isNeuronReduction()) {
                        groupEnv.add(Type::Uint32.addConst(), "batch", batched ? "blockIdx.y" : "0");
                        groupEnv.getStream() << "if(" << (batched ? "true" : ((batchSize > 1) ? "blockIdx.y == 0u" : "true")) << ")";
                        CodeStream::Scope b2(groupEnv.getStream());
                        EnvironmentGroupMergedField<CustomUpdateGroupMerged> batchEnv(groupEnv, c);
                        buildStandardEnvironment(batchEnv, batchSize);
                        const auto targets = genInitReductionTargets(batchEnv.getStream(), c, batchSize);
                        batchEnv.print("for(unsigned int idx = threadIdx.x; idx < $(num_neurons); idx += 256u)");
                        {
                            CodeStream::Scope b3(batchEnv.getStream());
                            EnvironmentGroupMergedField<CustomUpdateGroupMerged> loopEnv(batchEnv, c);
                            loopEnv.add(Type::Uint32.addConst(), "id", "idx");
                            c.generateCustomUpdate(loopEnv, batchSize, [&](auto &env, const auto&) { reduceOps(env, targets); });
                        }
                        for(const auto &r : targets) {
                            batchEnv.getStream() << "_lr" << r.name << " = gennmi_kernel::blockReduce" << ((r.access & VarAccessModeAttribute::SUM) ? "Sum" : "Max")
                                                 << "(_lr" << r.name << ");" << std::endl;
                        }
                        batchEnv.getStream() << "if(threadIdx.x == 0u)";
                        {
                            CodeStream::Scope b3(batchEnv.getStream());
                            for(const auto &r : targets) { batchEnv.printLine("group->" + r.name + "[" + r.index + "] = _lr" + r.name + ";"); }
                        }
                    }
                    else if(perElement) {
                        groupEnv.getStream() << "const unsigned int id = entry.firstId + threadIdx.x;" << std::endl;
                        groupEnv.add(Type::Uint32.addConst(), "id", "id");
                        groupEnv.add(Type::Uint32.addConst(), "batch", batched ? "blockIdx.y" : "0");
                        EnvironmentGroupMergedField<CustomUpdateGroupMerged> batchEnv(groupEnv, c);
                        buildStandardEnvironment(batchEnv, batchSize);
                        batchEnv.print("if(" + (batched ? std::string() : firstRowOnly) + "$(id) < $(num_neurons))");
                        CodeStream::Scope b2(batchEnv.getStream());
                        c.generateCustomUpdate(batchEnv, batchSize, [](auto&, auto&) {});
                    }
                    else {
                        // variables shared between the neurons of a population: one lane per batch
                        groupEnv.add(Type::Uint32.addConst(), "id", "0");
                        groupEnv.add(Type::Uint32.addConst(), "batch", batched ? "blockIdx.y" : "0");
                        groupEnv.getStream() << "if(" << (batched ? std::string() : firstRowOnly) << "threadIdx.x == 0u)";
                        CodeStream::Scope b2(groupEnv.getStream());
                        EnvironmentGroupMergedField<CustomUpdateGroupMerged> batchEnv(groupEnv, c);
                        buildStandardEnvironment(batchEnv, batchSize);
                        c.generateCustomUpdate(batchEnv, batchSize, [](auto&, auto&) {});
                    }
                    noteWrites(notes, c, "CustomUpdate", {});
                });
        }

        // ---- per-synapse custom updates
        std::ostringstream wuBody, wuArgs, wuParams, wuTables;
        size_t wuBlocks = 0;
        {
            CodeStream body(wuBody);
            EnvironmentLibrary lib(body, StandardLibrary::getMathsFunctions());
            EnvironmentExternal funcEnv(lib);
            funcEnv.add(model.getTimePrecision().addConst(), "t", "t");
            funcEnv.add(model.getTimePrecision().addConst(), "dt", Type::writeNumeric(model.getDT(), model.getTimePrecision()));
            modelMerged.genMergedCustomUpdateWUGroups(
                *this, memorySpaces, name,
                [&](auto &c)
                {
                    const auto &arch = c.getArchetype();
                    refuseRNG(arch);
                    const SynapseGroupInternal *sg = arch.getSynapseGroup();
                    const bool kernel = (sg->getMatrixType() & SynapseMatrixWeight::KERNEL);
                    const bool sparse = (sg->getMatrixType() & SynapseMatrixConnectivity::SPARSE);
                    if(!kernel && !sparse && !(sg->getMatrixType() & SynapseMatrixConnectivity::DENSE)) {
                        notGenerated("custom updates of matrices that are neither SPARSE, DENSE nor KERNEL (custom update '" + arch.getName() + "')");
                    }
                    const bool batched = (arch.getDims() & VarAccessDim::BATCH) && (batchSize > 1);
                    const bool batchReduction = arch.isBatchReduction();
                    const size_t firstBlock = wuBlocks;
                    const std::string starts = "gennmiCustomUpdateWU" + name + "Starts" + std::to_string(c.getIndex());
                    wuTables << "__device__ const uint32_t " << starts << "[] = {";
                    for(const auto &g : c.getGroups()) {
                        const SynapseGroupInternal *gsg = g.get().getSynapseGroup();
                        size_t size = 1;
                        if(kernel) { for(unsigned int k : gsg->getKernelSize()) { size *= k; } }
                        else { size = (size_t)gsg->getSrcNeuronGroup()->getNumNeurons() * getSynapticMatrixRowStride(*gsg); }
                        wuTables << wuBlocks << "u, ";
                        wuBlocks += (size + 255) / 256;
                        if(wuBlocks > 0x7FFFFFFFull) { notGenerated("custom updates over this many synapses in one update group"); }
                    }
                    wuTables << wuBlocks << "u};" << std::endl;
                    const std::string structArray = "mergedCustomUpdateWUGroup" + std::to_string(c.getIndex());
                    wuArgs << ", d_" << structArray;
                    wuParams << ", const MergedCustomUpdateWUGroup" << c.getIndex() << " *" << structArray;
                    const std::string idType = getSynapseIndexType(c).getName();

                    funcEnv.getStream() << "// merged custom WU update group " << c.getIndex() << std::endl;
                    funcEnv.getStream() << (firstBlock == 0 ? "if" : "else if") << "(blockIdx.x < " << wuBlocks << "u)";
                    CodeStream::Scope b(funcEnv.getStream());
                    funcEnv.getStream() << "const unsigned int gennmiGroup = gennmi_kernel::groupOfBlock(" << starts << ", " << c.getGroups().size() << "u, blockIdx.x);" << std::endl;
                    funcEnv.getStream() << "const auto *group = &" << structArray << "[gennmiGroup];" << std::endl;
                    funcEnv.getStream() << "const " << idType << " id = (" << idType << ")(blockIdx.x - " << starts << "[gennmiGroup]) * 256u + threadIdx.x;" << std::endl;

                    EnvironmentGroupMergedField<CustomUpdateWUGroupMerged> groupEnv(funcEnv, c);
                    buildSizeEnvironment(groupEnv);
                    groupEnv.add(getSynapseIndexType(c).addConst(), "id", "id");
                    if(!batchReduction) { groupEnv.add(Type::Uint32.addConst(), "batch", batched ? "blockIdx.y" : "0"); }
                    groupEnv.print("if(" + std::string((batched && !batchReduction) || batchSize == 1 ? "" : "blockIdx.y == 0u && ") + "$(id) < $(_size))");
                    CodeStream::Scope b2(groupEnv.getStream());
                    EnvironmentGroupMergedField<CustomUpdateWUGroupMerged> synEnv(groupEnv, c);
                    if(kernel) {
                        synEnv.add(Type::Uint32.addConst(), "id_kernel", "$(id)");
                    }
                    else if(sparse) {
                        synEnv.printLine("const unsigned int row = (unsigned int)($(id) / $(_row_stride));");
                        synEnv.printLine("const unsigned int col = (unsigned int)($(id) % $(_row_stride));");
                        synEnv.add(Type::Uint32.addConst(), "id_pre", "row");
                        synEnv.add(Type::Uint32.addConst(), "id_post", "$(_ind)[$(id)]");
                        synEnv.print("if(col < $(_row_length)[row])");
                        synEnv.getStream() << CodeStream::OB(2);
                    }
                    else {
                        synEnv.add(Type::Uint32.addConst(), "id_pre", "idPre", {synEnv.addInitialiser("const unsigned int idPre = (unsigned int)($(id) / $(_row_stride));")});
                        synEnv.add(Type::Uint32.addConst(), "id_post", "idPost", {synEnv.addInitialiser("const unsigned int idPost = (unsigned int)($(id) % $(_row_stride));")});
                    }
                    synEnv.add(getSynapseIndexType(c).addConst(), "id_syn", "$(id)");
                    const auto targets = genInitReductionTargets(synEnv.getStream(), c, batchSize, synEnv["id_syn"]);
                    if(batchReduction) {
                        synEnv.getStream() << "for(unsigned int batch = 0; batch < " << batchSize << "u; batch++)";
                        synEnv.getStream() << CodeStream::OB(1);
                        synEnv.add(Type::Uint32.addConst(), "batch", "batch");
                    }
                    {
                        EnvironmentGroupMergedField<CustomUpdateWUGroupMerged> batchEnv(synEnv, c);
                        buildStandardEnvironment(batchEnv, batchSize);
                        c.generateCustomUpdate(batchEnv, batchSize, [&](auto &env, auto&) { if(batchReduction) { reduceOps(env, targets); } });
                    }
                    if(batchReduction) {
                        synEnv.getStream() << CodeStream::CB(1);
                        for(const auto &r : targets) { synEnv.printLine("group->" + r.name + "[" + r.index + "] = _lr" + r.name + ";"); }
                    }
                    if(sparse && !kernel) { synEnv.getStream() << CodeStream::CB(2); }
                    noteWrites(notes, c, "CustomUpdateWU", {});
                });
        }

        // ---- per-synapse custom updates that also write the transpose of one variable (DENSE only, customUpdate.cc checks)
        std::ostringstream trBody, trArgs, trParams, trTables;
        size_t trBlocks = 0;
        {
            CodeStream body(trBody);
            EnvironmentLibrary lib(body, StandardLibrary::getMathsFunctions());
            EnvironmentExternal funcEnv(lib);
            funcEnv.add(model.getTimePrecision().addConst(), "t", "t");
            funcEnv.add(model.getTimePrecision().addConst(), "dt", Type::writeNumeric(model.getDT(), model.getTimePrecision()));
            modelMerged.genMergedCustomUpdateTransposeWUGroups(
                *this, memorySpaces, name,
                [&](auto &c)
                {
                    const auto &arch = c.getArchetype();
                    refuseRNG(arch);
                    const bool batched = (arch.getDims() & VarAccessDim::BATCH) && (batchSize > 1);
                    const size_t firstBlock = trBlocks;
                    const std::string starts = "gennmiCustomUpdateTranspose" + name + "Starts" + std::to_string(c.getIndex());
                    trTables << "__device__ const uint32_t " << starts << "[] = {";
                    for(const auto &g : c.getGroups()) {
                        const SynapseGroupInternal *gsg = g.get().getSynapseGroup();
                        trTables << trBlocks << "u, ";
                        trBlocks += (((size_t)gsg->getSrcNeuronGroup()->getNumNeurons() + 63) / 64) * (((size_t)gsg->getTrgNeuronGroup()->getNumNeurons() + 63) / 64);
                    }
                    trTables << trBlocks << "u};" << std::endl;
                    const std::string structArray = "mergedCustomUpdateTransposeWUGroup" + std::to_string(c.getIndex());
                    trArgs << ", d_" << structArray;
                    trParams << ", const MergedCustomUpdateTransposeWUGroup" << c.getIndex() << " *" << structArray;

                    funcEnv.getStream() << "// merged custom WU transpose update group " << c.getIndex() << std::endl;
                    funcEnv.getStream() << (firstBlock == 0 ? "if" : "else if") << "(blockIdx.x < " << trBlocks << "u)";
                    CodeStream::Scope b(funcEnv.getStream());
                    funcEnv.getStream() << "const unsigned int gennmiGroup = gennmi_kernel::groupOfBlock(" << starts << ", " << c.getGroups().size() << "u, blockIdx.x);" << std::endl;
                    funcEnv.getStream() << "const auto *group = &" << structArray << "[gennmiGroup];" << std::endl;
                    funcEnv.getStream() << "const unsigned int block = blockIdx.x - " << starts << "[gennmiGroup];" << std::endl;
                    funcEnv.getStream() << "const unsigned int tx = threadIdx.x & 63u, ty = threadIdx.x >> 6;" << std::endl;
                    // (an update that is not batched runs in the first of the grid's batch rows only; the condition is uniform
                    // over a work-group, as the barrier below needs)
                    funcEnv.getStream() << "if(" << ((batched || batchSize == 1) ? "true" : "blockIdx.y == 0u") << ")";
                    CodeStream::Scope b2(funcEnv.getStream());

                    EnvironmentGroupMergedField<CustomUpdateTransposeWUGroupMerged> groupEnv(funcEnv, c);
                    buildSizeEnvironment(groupEnv);
                    groupEnv.add(Type::Uint32.addConst(), "batch", batched ? "blockIdx.y" : "0");
                    EnvironmentGroupMergedField<CustomUpdateTransposeWUGroupMerged> batchEnv(groupEnv, c);
                    buildStandardEnvironment(batchEnv, batchSize);
                    const std::string transposeVar = c.addTransposeField(batchEnv);
                    batchEnv.printLine("const unsigned int numXBlocks = ($(num_post) + 63u) / 64u;");
                    batchEnv.printLine("const unsigned int blockX = block % numXBlocks, blockY = block / numXBlocks;");
                    {
                        CodeStream::Scope b3(batchEnv.getStream());
                        batchEnv.getStream() << "const unsigned int x = blockX * 64u + tx, y = blockY * 64u + ty;" << std::endl;
                        batchEnv.print("if(x < $(num_post))");
                        CodeStream::Scope b4(batchEnv.getStream());
                        batchEnv.print("for(unsigned int j = 0; j < 64u && (y + j) < $(num_pre); j += 4u)");
                        CodeStream::Scope b5(batchEnv.getStream());
                        EnvironmentGroupMergedField<CustomUpdateTransposeWUGroupMerged> synEnv(batchEnv, c);
                        synEnv.add(Type::Uint32.addConst(), "id_pre", "(y + j)");
                        synEnv.add(Type::Uint32.addConst(), "id_post", "x");
                        synEnv.add(Type::Uint32.addConst(), "id_syn", "idSyn", {synEnv.addInitialiser("const unsigned int idSyn = ((y + j) * $(num_post)) + x;")});
                        c.generateCustomUpdate(synEnv, batchSize,
                                               [&transposeVar](auto &env, const auto&) { env.printLine("gennmiTile[ty + j][tx] = $(" + transposeVar + ");"); });
                    }
                    batchEnv.getStream() << "__syncthreads();" << std::endl;
                    {
                        CodeStream::Scope b3(batchEnv.getStream());
                        batchEnv.getStream() << "const unsigned int x = blockY * 64u + tx, y = blockX * 64u + ty;" << std::endl;
                        batchEnv.print("if(x < $(num_pre))");
                        CodeStream::Scope b4(batchEnv.getStream());
                        batchEnv.print("for(unsigned int j = 0; j < 64u && (y + j) < $(num_post); j += 4u)");
                        CodeStream::Scope b5(batchEnv.getStream());
                        batchEnv.printLine("$(" + transposeVar + "_transpose)[" + (batched ? "$(_batch_offset) + " : "") + "((y + j) * $(num_pre)) + x] = gennmiTile[tx][ty + j];");
                    }
                    noteWrites(notes, c, "CustomUpdateTransposeWU", {transposeVar + "Transpose"});
                });
        }

        // ---- custom connectivity updates: a lane per row runs the row update code; add_synapse / remove_synapse and the
        // bookkeeping of every variable that lives on the synapses are GeNN's (generateUpdate).  Random numbers: a
        // counter-based generator per row and call (key = the model's seed, stream 6000 + the update's place in the model's
        // name-ordered list; the reference keeps a generator state per row in memory, backendSIMT.cc:1273-1305)
        std::ostringstream ccBody, ccArgs, ccParams, ccRemap;
        BlockTable ccTable;
        {
            CodeStream body(ccBody);
            EnvironmentLibrary lib(body, StandardLibrary::getMathsFunctions());
            EnvironmentLibrary rngLib(lib, simRNGFunctions);
            EnvironmentExternal funcEnv(rngLib);
            funcEnv.add(model.getTimePrecision().addConst(), "t", "t");
            funcEnv.add(model.getTimePrecision().addConst(), "dt", Type::writeNumeric(model.getDT(), model.getTimePrecision()));
            modelMerged.genMergedCustomConnectivityUpdateGroups(
                *this, memorySpaces, name,
                [&](auto &c)
                {
                    const auto &arch = c.getArchetype();
                    const size_t firstBlock = ccTable.numBlocks;
                    for(size_t g = 0; g < c.getGroups().size(); g++) {
                        const size_t blocks = ((size_t)c.getGroups()[g].get().getSynapseGroup()->getSrcNeuronGroup()->getNumNeurons() + 255) / 256;
                        for(size_t b = 0; b < blocks; b++) { ccTable.add(g, b * 256, b, blocks); }
                    }
                    const std::string structArray = "mergedCustomConnectivityUpdateGroup" + std::to_string(c.getIndex());
                    ccArgs << ", d_" << structArray;
                    ccParams << ", const MergedCustomConnectivityUpdateGroup" << c.getIndex() << " *" << structArray;
                    funcEnv.getStream() << "// merged custom connectivity update group " << c.getIndex() << std::endl;
                    funcEnv.getStream() << (firstBlock == 0 ? "if" : "else if") << "(blockIdx.x < " << ccTable.numBlocks << "u)";
                    CodeStream::Scope b(funcEnv.getStream());
                    funcEnv.getStream() << "const gennmi_kernel::BlockEntry entry = gennmiCustomConnectivityUpdate" << name << "Blocks[blockIdx.x];" << std::endl;
                    funcEnv.getStream() << "const auto *group = &" << structArray << "[entry.group];" << std::endl;
                    funcEnv.getStream() << "const unsigned int id = entry.firstId + threadIdx.x;" << std::endl;
                    EnvironmentGroupMergedField<CustomConnectivityUpdateGroupMerged> groupEnv(funcEnv, c);
                    buildStandardEnvironment(groupEnv);
                    groupEnv.print("if(id < $(num_pre))");
                    CodeStream::Scope b2(groupEnv.getStream());
                    EnvironmentGroupMergedField<CustomConnectivityUpdateGroupMerged> rowEnv(groupEnv, c);
                    rowEnv.add(Type::Uint32.addConst(), "id_pre", "id");
                    if(Utils::isRNGRequired(arch.getRowUpdateCodeTokens())) {
                        rowEnv.addField(Type::Uint32.addConst(), "_rng_stream", Type::Uint32, "rngStream",
                                        [&model](const CustomConnectivityUpdateInternal &g, size_t)
                                        {
                                            return Type::NumericValue((uint64_t)(6000 + std::distance(model.getCustomConnectivityUpdates().cbegin(), model.getCustomConnectivityUpdates().find(g.getName()))));
                                        });
                        rowEnv.add(Type::Uint32, "_rng", "gennmiRng",
                                   {rowEnv.addInitialiser("gennmi_kernel::Rng gennmiRng = gennmi_kernel::rngBegin(gennmiSeed, $(_rng_stream), (unsigned long long)id, gennmiStep);")});
                    }
                    c.generateUpdate(*this, rowEnv, batchSize);
                });
        }
        // ... after which the column views of projections that learn from postsynaptic spikes are rebuilt by the device library
        // (deterministic order, as at initialisation; the reference has a kernel of its own for this, backendSIMT.cc:1307-1400)
        {
            CodeStream remap(ccRemap);
            EnvironmentLibrary lib(remap, StandardLibrary::getMathsFunctions());
            EnvironmentExternal funcEnv(lib);
            modelMerged.genMergedCustomConnectivityRemapUpdateGroups(
                *this, memorySpaces, name,
                [&](auto &c)
                {
                    funcEnv.getStream() << "for(unsigned int g = 0; g < " << c.getGroups().size() << "u; g++)";
                    CodeStream::Scope b(funcEnv.getStream());
                    funcEnv.getStream() << "const auto *group = &mergedCustomConnectivityRemapUpdateGroup" << c.getIndex() << "[g];" << std::endl;
                    EnvironmentGroupMergedField<CustomConnectivityRemapUpdateGroupMerged> env(funcEnv, c);
                    buildStandardEnvironment(env);
                    env.printLine("GENNMI_CHECK(gennmi_build_remap($(num_pre), $(num_post), $(_row_stride), $(_col_stride), gennmiDev($(_row_length)), gennmiDev($(_ind)), "
                                  "gennmiDev($(_col_length)), gennmiDev($(_remap))));");
                });
        }

        // ---- host update code of custom connectivity updates: plain host code over the arrays' host buffers, run before the
        // group's kernels; its pushXToDevice / pullXFromDevice are copies between a host buffer and the device buffer behind it
        std::ostringstream ccHost;
        {
            CodeStream hostCode(ccHost);
            EnvironmentLibrary lib(hostCode, StandardLibrary::getMathsFunctions());
            EnvironmentExternal funcEnv(lib);
            funcEnv.add(model.getTimePrecision().addConst(), "t", "t");
            funcEnv.add(Type::Uint32.addConst(), "batch", "0");
            funcEnv.add(model.getTimePrecision().addConst(), "dt", Type::writeNumeric(model.getDT(), model.getTimePrecision()));
            modelMerged.genMergedCustomConnectivityHostUpdateGroups(*this, memorySpaces, name, [&](auto &c) { c.generateUpdate(*this, funcEnv); });
        }

        // ---- kernels and the host function of this update group
        const std::string signature = "(" + timeType + " t";
        if(neuronTable.numBlocks > 0) {
            device << "__device__ const gennmi_kernel::BlockEntry gennmiCustomUpdate" << name << "Blocks[] = {" << std::endl << neuronTable.entries.str() << "{0u, 0u, 0u, 0u}};" << std::endl;
            device << "__global__ __launch_bounds__(256) void gennmiCustomUpdate" << name << "Kernel" << signature << neuronParams.str() << ")";
            CodeStream::Scope b(device);
            device << neuronBody.str();
        }
        if(wuBlocks > 0) {
            device << wuTables.str();
            device << "__global__ __launch_bounds__(256) void gennmiCustomUpdateWU" << name << "Kernel" << signature << wuParams.str() << ")";
            CodeStream::Scope b(device);
            device << wuBody.str();
        }
        if(ccTable.numBlocks > 0) {
            device << "__device__ const gennmi_kernel::BlockEntry gennmiCustomConnectivityUpdate" << name << "Blocks[] = {" << std::endl << ccTable.entries.str() << "{0u, 0u, 0u, 0u}};" << std::endl;
            device << "__global__ __launch_bounds__(256) void gennmiCustomConnectivityUpdate" << name << "Kernel" << signature << ", unsigned long long gennmiSeed, unsigned long long gennmiStep" << ccParams.str() << ")";
            CodeStream::Scope b(device);
            device << ccBody.str();
        }
        if(trBlocks > 0) {
            device << trTables.str();
            device << "__global__ __launch_bounds__(256) void gennmiCustomUpdateTranspose" << name << "Kernel" << signature << trParams.str() << ")";
            CodeStream::Scope b(device);
            device << "__shared__ " << model.getPrecision().getName() << " gennmiTile[64][65];" << std::endl;
            device << trBody.str();
        }
        host << "void update" << name << "(unsigned long long timestep)";
        {
            CodeStream::Scope b(host);
            host << "gennmiEnsureFinalised();" << std::endl;
            // (beside the library's kernels: steps still queued run first; the launches below go to the null stream, which is
            // ordered against the runner's stream in both directions)
            if(!m_GeneratedKernels) { host << "GENNMI_CHECK(gennmi_flush());" << std::endl; }
            host << "const " << timeType << " t = timestep * " << Type::writeNumeric(model.getDT(), model.getTimePrecision()) << ";" << std::endl;
            const std::string grid = ", " + std::to_string(batchSize) + "), dim3(256), 0, 0>>>(t";
            const bool timing = model.isTimingEnabled();
            if(timing) { host << "hipEventRecord(customUpdate" << name << "Start, 0);" << std::endl; }
            host << ccHost.str();
            if(ccTable.numBlocks > 0) {
                // (connectivity first, like the reference: single_threaded_cpu/backend.cc:824-860; the generator's step counts this group's calls)
                host << "static unsigned long long gennmiCalls = 0;" << std::endl;
                host << "gennmiCustomConnectivityUpdate" << name << "Kernel<<<dim3(" << ccTable.numBlocks << ", 1), dim3(256), 0, 0>>>(t, "
                     << ((model.getSeed() != 0) ? (std::to_string(model.getSeed()) + "ull") : std::string("gennmiRandomSeed()")) << ", gennmiCalls++" << ccArgs.str() << ");" << std::endl;
                host << ccRemap.str();
            }
            if(neuronTable.numBlocks > 0) { host << "gennmiCustomUpdate" << name << "Kernel<<<dim3(" << neuronTable.numBlocks << grid << neuronArgs.str() << ");" << std::endl; }
            if(wuBlocks > 0) { host << "gennmiCustomUpdateWU" << name << "Kernel<<<dim3(" << wuBlocks << grid << wuArgs.str() << ");" << std::endl; }
            if(timing) { host << "hipEventRecord(customUpdate" << name << "Stop, 0);" << std::endl << "hipEventRecord(customUpdate" << name << "TransposeStart, 0);" << std::endl; }
            if(trBlocks > 0) { host << "gennmiCustomUpdateTranspose" << name << "Kernel<<<dim3(" << trBlocks << grid << trArgs.str() << ");" << std::endl; }
            if(timing) { host << "hipEventRecord(customUpdate" << name << "TransposeStop, 0);" << std::endl; }
            host << "if(hipGetLastError() != hipSuccess) { throw std::runtime_error(\"update" << name << ": kernel launch failed\"); }" << std::endl;
            host << notes.str();
            if(timing) {
                // (these counters are not part of stepTime: read here, after the group's kernels have finished, backendCUDAHIP.cc:826-856)
                host << "GENNMI_CHECK(gennmi_synchronize());" << std::endl;
                host << "float tmp = 0.0f;" << std::endl;
                host << "if(hipEventElapsedTime(&tmp, customUpdate" << name << "Start, customUpdate" << name << "Stop) == hipSuccess) { customUpdate" << name << "Time += tmp / 1000.0; }" << std::endl;
                host << "if(hipEventElapsedTime(&tmp, customUpdate" << name << "TransposeStart, customUpdate" << name << "TransposeStop) == hipSuccess) { customUpdate" << name << "TransposeTime += tmp / 1000.0; }" << std::endl;
            }
        }
        host << std::endl;
    }

    // struct definitions, host arrays and push functions (GeNN's own), then the device copies
    modelMerged.genMergedCustomUpdateStructs(os, *this);
    modelMerged.genMergedCustomUpdateWUStructs(os, *this);
    modelMerged.genMergedCustomUpdateTransposeWUStructs(os, *this);
    modelMerged.genMergedCustomConnectivityUpdateStructs(os, *this);
    modelMerged.genMergedCustomConnectivityRemapUpdateStructs(os, *this);
    modelMerged.genMergedCustomConnectivityHostUpdateStructs(os, *this);
    modelMerged.genMergedCustomConnectivityHostUpdateStructArrayPush(os, *this);
    modelMerged.genMergedCustomConnectivityUpdateHostStructArrayPush(os, *this);
    modelMerged.genMergedCustomConnectivityRemapUpdateHostStructArrayPush(os, *this);
    modelMerged.genMergedCustomUpdateHostStructArrayPush(os, *this);
    modelMerged.genMergedCustomUpdateWUHostStructArrayPush(os, *this);
    modelMerged.genMergedCustomUpdateTransposeWUHostStructArrayPush(os, *this);
    preambleHandler(os);
    for(const auto &g : modelMerged.getMergedCustomUpdateGroups()) { genDeviceStructArray(decl, upload, *this, g, "CustomUpdate"); }
    for(const auto &g : modelMerged.getMergedCustomUpdateWUGroups()) { genDeviceStructArray(decl, upload, *this, g, "CustomUpdateWU"); }
    for(const auto &g : modelMerged.getMergedCustomUpdateTransposeWUGroups()) { genDeviceStructArray(decl, upload, *this, g, "CustomUpdateTransposeWU"); }
    for(const auto &g : modelMerged.getMergedCustomConnectivityUpdateGroups()) { genDeviceStructArray(decl, upload, *this, g, "CustomConnectivityUpdate"); }
    os << declStream.str();
    os << std::endl;
    os << "void gennmiUploadCustomUpdateGroups()";
    {
        CodeStream::Scope b(os);
        os << uploadStream.str();
    }
    os << std::endl;
    os << deviceStream.str();
    os << std::endl;
    os << hostStream.str();
}
}   // namespace GeNN::CodeGenerator::MI355X
