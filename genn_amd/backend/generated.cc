// GeNN::CodeGenerator::MI355X::Backend — generated kernels.
//
// For models whose snippets the device library does not implement, the step's device code is generated: the model's own
// code strings — sim / threshold / reset code, postsynaptic and current-source code, weight-update code with its pre and
// post variables — are printed by GeNN's environments and pretty-printer (the transpiler stays in libgenn:
// NeuronUpdateGroupMerged::generateNeuronUpdate, PresynapticUpdateGroupMerged::generateSpikeUpdate, ...) into the
// skeletons emitted here.  Every module that holds device code is compiled twice by the runner's Makefile: by the host
// compiler, which sees the merged-group structs, the host arrays and the host functions (the kernels are hidden from it), and
// by `hipcc --genco`, which turns the kernels into a gfx950 code object that is embedded in the module's object file.  The host
// functions load and launch that code object through the device library's C ABI (gennmi_program_*, include/genn_mi355x.h): the
// runner contains no launch syntax and no HIP call, and a model's steps can be noted and replayed from a captured graph.
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

// Arguments of one generated kernel beyond the launch header: a struct that both passes of the module see.  Every kernel
// gets the look-back area and error flag of ordered compactions, the seed of counter-based random numbers, and a pointer to
// the device copy of each merged group's struct array it walks.
struct KernelArgs
{
    explicit KernelArgs(const std::string &kernelName) : name(kernelName) {}
    std::string name;
    std::ostringstream members, unpack, fill;
    void add(const std::string &type, const std::string &structArray)
    {
        members << "    const " << type << " *" << structArray << ";" << std::endl;
        unpack << "const " << type << " *" << structArray << " = gennmiArgs." << structArray << ";" << std::endl;
        fill << "a." << structArray << " = d_" << structArray << "; ";
    }
    void addWord(const std::string &member, const std::string &hostValue)     // a device word of the launch's own
    {
        members << "    uint32_t *" << member << ";" << std::endl;
        fill << "a." << member << " = " << hostValue << "; ";
    }
    std::string type() const { return "G" + name.substr(1) + "Args"; }      // gennmiXKernel -> GennmiXKernelArgs
    void define(CodeStream &os) const
    {
        os << "struct " << type() << std::endl << "{" << std::endl;
        os << "    unsigned long long *agg;" << std::endl << "    uint32_t *error;" << std::endl << "    unsigned long long seed;" << std::endl;
        os << members.str() << "};" << std::endl;
    }
    // device pass: signature and the statements that give the kernel's body the names it was written with
    void open(CodeStream &os, const std::string &timeType, const std::string &attributes = "__launch_bounds__(256) ") const
    {
        os << "extern \"C\" __global__ " << attributes << "void " << name << "(gennmi_launch_header_t gennmiLaunch, " << type() << " gennmiArgs)";
        os << CodeStream::OB(9000);
        os << "const gennmi_step_entry_t gennmiEntry = gennmi_kernel::stepEntry(gennmiLaunch);" << std::endl;
        os << "const " << timeType << " t = (" << timeType << ")gennmiEntry.t;" << std::endl;
        os << "const unsigned int recordingTimestep = gennmiEntry.recordingTimestep;" << std::endl;
        os << "const uint32_t gennmiTag = gennmiEntry.tag;" << std::endl;
        os << "const unsigned long long gennmiStep = gennmiEntry.step;" << std::endl;
        os << "unsigned long long *gennmiAgg = gennmiArgs.agg;" << std::endl;
        os << "uint32_t *gennmiError = gennmiArgs.error;" << std::endl;
        os << "const unsigned long long gennmiSeed = gennmiArgs.seed;" << std::endl;
        os << unpack.str();
    }
    void close(CodeStream &os) const { os << CodeStream::CB(9000); }
    // host pass: the statements that fill an argument block `a` (agg / seed as given)
    std::string fillBlock(const std::string &agg, const std::string &seed) const
    {
        return type() + " a{}; a.agg = " + agg + "; a.error = gennmiProgramError; a.seed = " + seed + "; " + fill.str();
    }
    // host pass: looks the kernel up in `module` and appends it to a phase of the program
    void addToPhase(CodeStream &os, const std::string &phase, size_t gridX, size_t gridY, unsigned int block, int timer,
                    const std::string &agg, const std::string &seed) const
    {
        CodeStream::Scope b(os);
        os << "uint32_t k = 0;" << std::endl;
        os << "GENNMI_CHECK(gennmi_program_get_kernel(gennmiProgram, module, \"" << name << "\", &k));" << std::endl;
        os << fillBlock(agg, seed) << std::endl;
        os << "GENNMI_CHECK(gennmi_program_add_launch(gennmiProgram, " << phase << ", k, " << gridX << "u, " << gridY << "u, " << block << "u, &a, sizeof(a), " << timer << "));" << std::endl;
    }
};

// device copy of a merged group's struct array: declaration, and the statements that translate and upload it
template<typename G>
void genDeviceStructArray(CodeStream &decl, CodeStream &upload, CodeStream &release, const BackendBase &backend, const G &g, const std::string &name,
                          bool shared = false)
{
    const std::string type = "Merged" + name + "Group" + std::to_string(g.getIndex());
    const std::string host = "merged" + name + "Group" + std::to_string(g.getIndex());
    const std::string dev = "d_" + host;
    const size_t count = g.getGroups().size();
    decl << (shared ? "" : "static ") << type << " *" << dev << " = nullptr;" << std::endl;     // (shared: another module's kernel walks the array too)
    release << "if(" << dev << ") { gennmi_free(" << dev << "); " << dev << " = nullptr; }" << std::endl;
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

    std::ostringstream kernelStream, declStream, uploadStream, releaseStream;
    CodeStream kernel(kernelStream), decl(declStream), upload(uploadStream), release(releaseStream);
    BlockTable table;
    KernelArgs neuronKernel("gennmiNeuronUpdateKernel"), prevKernel("gennmiPrevSpikeTimeKernel"), queueKernel("gennmiSpikeQueueUpdateKernel");

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
            neuronKernel.add("MergedNeuronUpdateGroup" + std::to_string(n.getIndex()), structArray);

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
                               "gennmiTag, gennmiError, gennmiLaunch.spinLimit);");
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
                                      "blockIdx.x - entry.blockInGroup, " + region + ", " + region + " + gridDim.x, gennmiTag, gennmiError, gennmiLaunch.spinLimit);");
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
    std::ostringstream prevStream;
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
                prevKernel.add("MergedNeuronPrevSpikeTimeUpdateGroup" + std::to_string(n.getIndex()), structArray);
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
    std::ostringstream queueStream;
    if(anyDelaySlots) {
        CodeStream queue(queueStream);
        EnvironmentLibrary queueLib(queue, StandardLibrary::getMathsFunctions());
        EnvironmentExternal queueEnv(queueLib);
        modelMerged.genMergedNeuronSpikeQueueUpdateGroups(
            *this, memorySpaces,
            [&](auto &n)
            {
                const std::string structArray = "mergedNeuronSpikeQueueUpdateGroup" + std::to_string(n.getIndex());
                queueKernel.add("MergedNeuronSpikeQueueUpdateGroup" + std::to_string(n.getIndex()), structArray);
                queueEnv.getStream() << "for(unsigned int g = threadIdx.x; g < " << n.getGroups().size() << "u; g += blockDim.x)";
                CodeStream::Scope b(queueEnv.getStream());
                queueEnv.getStream() << "const auto *group = &" << structArray << "[g];" << std::endl;
                EnvironmentGroupMergedField<NeuronSpikeQueueUpdateGroupMerged> groupEnv(queueEnv, n);
                buildStandardEnvironment(groupEnv, batchSize);
                n.genSpikeQueueUpdate(groupEnv, batchSize);
            });
    }

    // Dendritic-delay ring pointers: moved on for the next step by the last work-group of this kernel to finish (the reference
    // launches a one-thread-per-group kernel at the start of updateSynapses, synapseUpdateGroupMerged.cc:480-483; every read of a
    // pointer in this step lies before its work-group's arrival at the counter, and the next kernel starts after this one ends)
    std::ostringstream delayStream;
    bool anyDenDelay = false;
    {
        CodeStream delayCode(delayStream);
        EnvironmentLibrary delayLib(delayCode, StandardLibrary::getMathsFunctions());
        EnvironmentExternal delayEnv(delayLib);
        modelMerged.genMergedSynapseDendriticDelayUpdateGroups(
            *this, memorySpaces,
            [&](auto &sg)
            {
                anyDenDelay = true;
                const std::string structArray = "mergedSynapseDendriticDelayUpdateGroup" + std::to_string(sg.getIndex());
                neuronKernel.add("MergedSynapseDendriticDelayUpdateGroup" + std::to_string(sg.getIndex()), structArray);
                delayEnv.getStream() << "for(unsigned int g = threadIdx.x; g < " << sg.getGroups().size() << "u; g += blockDim.x)";
                CodeStream::Scope b(delayEnv.getStream());
                delayEnv.getStream() << "const auto *group = &" << structArray << "[g];" << std::endl;
                EnvironmentGroupMergedField<SynapseDendriticDelayUpdateGroupMerged> groupEnv(delayEnv, sg);
                buildStandardEnvironment(groupEnv, 1);
                sg.generateSynapseUpdate(groupEnv);
            });
    }
    if(anyDenDelay && table.numBlocks > 0) { neuronKernel.addWord("finished", "gennmiNeuronFinished"); }

    // struct definitions (both passes), then the host arrays and their push functions (GeNN's own) for the host pass
    const bool timing = model.isTimingEnabled();
    const std::string seed = anyRNG ? ((model.getSeed() != 0) ? (std::to_string(model.getSeed()) + "ull") : std::string("gennmiRandomSeed()")) : std::string("0ull");
    os << "#define GENNMI_DEVICE_MODULE 1      // the Makefile builds a gfx950 code object from this file as well" << std::endl;
    modelMerged.genMergedNeuronUpdateGroupStructs(os, *this);
    if(anyDelaySlots) { modelMerged.genMergedNeuronSpikeQueueUpdateStructs(os, *this); }
    if(anyPrevTimes) { modelMerged.genMergedNeuronPrevSpikeTimeUpdateStructs(os, *this); }
    if(anyDenDelay) { modelMerged.genMergedSynapseDendriticDelayUpdateStructs(os, *this); }
    neuronKernel.define(os);
    if(anyDelaySlots) { queueKernel.define(os); }
    if(anyPrevTimes) { prevKernel.define(os); }
    os << std::endl;

    // ---- device pass
    os << "#ifdef __HIPCC__" << std::endl;
    os << "__device__ const gennmi_kernel::BlockEntry gennmiNeuronBlocks[] = {" << std::endl << table.entries.str() << "{0u, 0u, 0u, 0u}};" << std::endl;
    if(anyPrevTimes) {
        os << "__device__ const gennmi_kernel::BlockEntry gennmiPrevSpikeTimeBlocks[] = {" << std::endl << prevTable.entries.str() << "{0u, 0u, 0u, 0u}};" << std::endl;
        prevKernel.open(os, timeType);
        os << prevStream.str();
        prevKernel.close(os);
    }
    if(anyDelaySlots) {
        queueKernel.open(os, timeType, "");
        os << queueStream.str();
        queueKernel.close(os);
    }
    os << std::endl;
    neuronKernel.open(os, timeType);
    os << kernelStream.str();
    if(anyDenDelay && table.numBlocks > 0) {
        os << "// the last work-group to get here moves the dendritic-delay ring pointers on for the next step" << std::endl;
        os << "__shared__ bool gennmiLastToFinish;" << std::endl;
        os << "__syncthreads();" << std::endl;
        os << "if(threadIdx.x == 0u)";
        {
            CodeStream::Scope b(os);
            // counted in two levels, sixteen work-groups to a word and one word per cache line: atomics on one address complete
            // one after the other (about 8 ns each), and every work-group waits for the answer to its own
            os << "const unsigned int linear = blockIdx.y * gridDim.x + blockIdx.x, total = gridDim.x * gridDim.y;" << std::endl;
            os << "const unsigned int group = linear >> 4, groups = (total + 15u) >> 4;" << std::endl;
            os << "const unsigned int inGroup = (total - (group << 4) < 16u) ? total - (group << 4) : 16u;" << std::endl;
            os << "uint32_t *groupWord = gennmiArgs.finished + 32u * (1u + group);" << std::endl;
            os << "bool last = false;" << std::endl;
            os << "if(__hip_atomic_fetch_add(groupWord, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == inGroup - 1u)";
            {
                CodeStream::Scope b2(os);
                os << "__hip_atomic_store(groupWord, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);" << std::endl;
                os << "if(__hip_atomic_fetch_add(gennmiArgs.finished, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == groups - 1u)";
                {
                    CodeStream::Scope b3(os);
                    os << "__hip_atomic_store(gennmiArgs.finished, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);" << std::endl;
                    os << "last = true;" << std::endl;
                }
            }
            os << "gennmiLastToFinish = last;" << std::endl;
        }
        os << "__syncthreads();" << std::endl;
        os << "if(gennmiLastToFinish)";
        {
            CodeStream::Scope b(os);
            os << delayStream.str();
        }
    }
    neuronKernel.close(os);
    os << std::endl;

    // ---- host pass
    os << "#else" << std::endl;
    modelMerged.genMergedNeuronUpdateGroupHostStructArrayPush(os, *this);
    if(anyDelaySlots) { modelMerged.genMergedNeuronSpikeQueueUpdateHostStructArrayPush(os, *this); }
    if(anyPrevTimes) { modelMerged.genMergedNeuronPrevSpikeTimeUpdateHostStructArrayPush(os, *this); }
    preambleHandler(os);
    for(const auto &n : modelMerged.getMergedNeuronUpdateGroups()) {
        genDeviceStructArray(decl, upload, release, *this, n, "NeuronUpdate");
    }
    if(anyDelaySlots) {
        for(const auto &n : modelMerged.getMergedNeuronSpikeQueueUpdateGroups()) { genDeviceStructArray(decl, upload, release, *this, n, "NeuronSpikeQueueUpdate"); }
    }
    if(anyPrevTimes) {
        for(const auto &n : modelMerged.getMergedNeuronPrevSpikeTimeUpdateGroups()) { genDeviceStructArray(decl, upload, release, *this, n, "NeuronPrevSpikeTimeUpdate"); }
    }
    os << declStream.str();
    os << "static unsigned long long *gennmiNeuronAgg = nullptr;" << std::endl;
    if(anyDenDelay) {
        os << "static uint32_t *gennmiNeuronFinished = nullptr;     // work-groups of the running neuron update that have finished" << std::endl;
        for(const auto &g : modelMerged.getMergedSynapseDendriticDelayUpdateGroups()) {
            os << "extern MergedSynapseDendriticDelayUpdateGroup" << g.getIndex() << " *d_mergedSynapseDendriticDelayUpdateGroup" << g.getIndex() << ";      // (uploaded by the synapse module)" << std::endl;
        }
    }
    os << "extern \"C\" const unsigned char gennmi_neuronUpdate_image[];" << std::endl;
    os << "extern \"C\" const unsigned char gennmi_neuronUpdate_image_end[];" << std::endl;
    os << std::endl;
    os << "void gennmiUploadNeuronGroups()";
    {
        CodeStream::Scope b(os);
        os << uploadStream.str();
        // (the first time: the look-back words of the ordered compactions, then the launches of updateNeurons(), in the order of
        // the reference's function, backendCUDAHIP.cc:386-420: previous spike times, ring pointers of the spike queues, the update)
        os << "if(!gennmiNeuronAgg)";
        {
            CodeStream::Scope b2(os);
            os << "void *p = nullptr;" << std::endl;
            os << "GENNMI_CHECK(gennmi_malloc(&p, " << 2 * std::max<size_t>(1, table.numBlocks) * batchSize * (1 + maxEventGroups) << " * sizeof(unsigned long long)));" << std::endl;
            os << "GENNMI_CHECK(gennmi_memset(p, 0, " << 2 * std::max<size_t>(1, table.numBlocks) * batchSize * (1 + maxEventGroups) << " * sizeof(unsigned long long)));" << std::endl;
            os << "gennmiNeuronAgg = (unsigned long long*)p;" << std::endl;
            if(anyDenDelay) {
                const size_t finishedWords = 32 * (2 + (std::max<size_t>(1, table.numBlocks) * batchSize + 15) / 16);       // (a cache line per word: see the kernel's end)
                os << "GENNMI_CHECK(gennmi_malloc(&p, " << finishedWords << " * sizeof(uint32_t)));" << std::endl;
                os << "GENNMI_CHECK(gennmi_memset(p, 0, " << finishedWords << " * sizeof(uint32_t)));" << std::endl;
                os << "gennmiNeuronFinished = (uint32_t*)p;" << std::endl;
            }
            os << "uint32_t module = 0;" << std::endl;
            os << "GENNMI_CHECK(gennmi_program_load_module(gennmiProgram, gennmi_neuronUpdate_image, (size_t)(gennmi_neuronUpdate_image_end - gennmi_neuronUpdate_image), &module));" << std::endl;
            if(anyPrevTimes) { prevKernel.addToPhase(os, "GENNMI_PHASE_NEURONS", prevTable.numBlocks, batchSize, 256, -1, "nullptr", "0ull"); }
            if(anyDelaySlots) { queueKernel.addToPhase(os, "GENNMI_PHASE_NEURONS", 1, 1, 64, -1, "nullptr", "0ull"); }
            if(table.numBlocks > 0) { neuronKernel.addToPhase(os, "GENNMI_PHASE_NEURONS", table.numBlocks, batchSize, 256, timing ? timerId("neuronUpdate") : -1, "gennmiNeuronAgg", seed); }
        }
    }
    os << std::endl;
    os << "void gennmiFreeNeuronGroups()";
    {
        CodeStream::Scope b(os);
        os << "if(gennmiNeuronAgg) { gennmi_free(gennmiNeuronAgg); gennmiNeuronAgg = nullptr; }" << std::endl;
        if(anyDenDelay) { os << "if(gennmiNeuronFinished) { gennmi_free(gennmiNeuronFinished); gennmiNeuronFinished = nullptr; }" << std::endl; }
        os << releaseStream.str();
    }
    os << std::endl;
    // the time, the recording row, the generator's step (calls of updateNeurons so far) and the look-back tag of the call travel
    // in the launch header; a bounded wait of the compaction that expires raises the program's error flag, which the library
    // reports from the next call that waits for the device (whatever the timing setting)
    os << "void updateNeurons(" << model.getTimePrecision().getName() << " t";
    if(recording) { os << ", unsigned int recordingTimestep"; }
    os << ")";
    {
        CodeStream::Scope b(os);
        os << "gennmiEnsureFinalised();" << std::endl;
        os << "GENNMI_CHECK(gennmi_program_update(gennmiProgram, GENNMI_PHASE_NEURONS, (double)t, " << (recording ? "recordingTimestep" : "0u") << "));" << std::endl;
    }
    os << "#endif" << std::endl;
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

    std::ostringstream declStream, uploadStream, releaseStream;
    CodeStream decl(declStream), upload(uploadStream), release(releaseStream);

    // every kernel's body, arguments and block table
    struct KernelText
    {
        explicit KernelText(const std::string &name) : args(name) {}
        std::ostringstream body;
        KernelArgs args;
        BlockTable table;
    };
    KernelText delay("gennmiDendriticDelayUpdateKernel"), dynamics("gennmiSynapseDynamicsKernel"), pre("gennmiPresynapticUpdateKernel"), post("gennmiPostsynapticUpdateKernel");
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
                    dynamics.args.add("MergedSynapseDynamicsGroup" + std::to_string(s.getIndex()), structArray);

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
                    delay.args.add("MergedSynapseDendriticDelayUpdateGroup" + std::to_string(sg.getIndex()), structArray);
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
    auto presynapticBlocks = [this](const SynapseGroupInternal &sg) -> size_t
    {
        const auto matrix = sg.getMatrixType();
        const size_t rowLen = (matrix & SynapseMatrixConnectivity::PROCEDURAL) ? sg.getNumThreadsPerSpike()
                              : (matrix & SynapseMatrixConnectivity::DENSE) ? sg.getTrgNeuronGroup()->getNumNeurons() : getSynapticMatrixRowStride(sg);
        return std::clamp<size_t>((sg.getSrcNeuronGroup()->getNumNeurons() * ((rowLen + 63) / 64) + 255) / 256, 1, 128);
    };
    double presynapticScale = 1.0;
    {
        size_t wanted = 0;
        for(const auto &sg : model.getSynapseGroups()) {
            if(sg.second.isPreSpikeRequired() || sg.second.isPreSpikeEventRequired()) { wanted += presynapticBlocks(sg.second); }
        }
        const char *envRound = std::getenv("GENNMI_GENERATED_PRESYN_BLOCKS_PER_CU");
        // (work-groups of 256 threads per compute unit that all projections share; the full microcircuit through
        // Runtime::stepTime with 1 / 2 / 4 / 8 / 16 / 32: 38.2 / 26.8 / 20.6 / 18.3 / 17.8 / 18.0 us per step)
        const size_t oneRound = 256 * (envRound ? (size_t)std::max(1, std::atoi(envRound)) : 16);
        if(wanted > oneRound) { presynapticScale = (double)oneRound / (double)wanted; }
    }
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
                        // enough wavefronts for ~1.5 % of the source population firing in one step, at most 128 work-groups; a model of
                        // many projections shares one round of the chip between them in that proportion (a work-group that finds no
                        // spike leaves at once, but thousands of them still take microseconds to come and go)
                        const size_t blocks = std::max<size_t>(1, (size_t)((double)presynapticBlocks(sg) * presynapticScale));
                        for(size_t b = 0; b < blocks; b++) { pre.table.add(g, 0, b, blocks); }
                    }
                    const std::string structArray = "mergedPresynapticUpdateGroup" + std::to_string(s.getIndex());
                    pre.args.add("MergedPresynapticUpdateGroup" + std::to_string(s.getIndex()), structArray);

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
                        // (the queue entry of an item is asked for one item ahead, the first one together with the count: the queue
                        // always holds num_pre entries, so any index below that is readable, and an item's chain of dependent loads
                        // is row -> synapses instead of count -> entry -> row -> synapses)
                        groupEnv.getStream() << "unsigned long long item = entry.blockInGroup * 4u + (threadIdx.x / 64u);" << std::endl;
                        groupEnv.printLine("unsigned int spikeNext = (unsigned int)min(item / chunksPerRow, (unsigned long long)($(num_pre) - 1u));");
                        groupEnv.printLine("unsigned int idPreNext = $(_src_spk" + suffix + ")[" + s.getPreVarIndex(preDelay, batchSize, VarAccessDim::BATCH | VarAccessDim::ELEMENT, "spikeNext") + "];");
                        groupEnv.printLine("const unsigned int numSpikes = $(_src_spk_cnt" + suffix + ")[" + s.getPreSlot(preDelay, batchSize) + "];");
                        groupEnv.getStream() << "const unsigned long long numItems = (unsigned long long)numSpikes * chunksPerRow;" << std::endl;
                        groupEnv.getStream() << "while(item < numItems)";
                        CodeStream::Scope b2(groupEnv.getStream());
                        EnvironmentGroupMergedField<PresynapticUpdateGroupMerged> synEnv(groupEnv, s);
                        synEnv.getStream() << "const unsigned int spike = (unsigned int)(item / chunksPerRow);" << std::endl;
                        synEnv.getStream() << "const unsigned int j = (unsigned int)(item % chunksPerRow) * 64u + (threadIdx.x & 63u);" << std::endl;
                        synEnv.getStream() << "const unsigned int idPre = idPreNext;" << std::endl;
                        synEnv.getStream() << "item += numWaves;" << std::endl;
                        synEnv.printLine("spikeNext = (unsigned int)min(item / chunksPerRow, (unsigned long long)($(num_pre) - 1u));");
                        synEnv.printLine("idPreNext = $(_src_spk" + suffix + ")[" + s.getPreVarIndex(preDelay, batchSize, VarAccessDim::BATCH | VarAccessDim::ELEMENT, "spikeNext") + "];");
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
                    post.args.add("MergedPostsynapticUpdateGroup" + std::to_string(s.getIndex()), structArray);

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

    // struct definitions (both passes), then the kernels (device pass) or the host arrays, push functions and updateSynapses() (host pass)
    const bool anyDelay = delay.table.numBlocks > 0, anyPre = pre.table.numBlocks > 0, anyPost = post.table.numBlocks > 0, anyDynamics = dynamics.table.numBlocks > 0;
    const bool timing = model.isTimingEnabled();
    const std::string seed = anySynapseRNG ? ((model.getSeed() != 0) ? (std::to_string(model.getSeed()) + "ull") : std::string("gennmiRandomSeed()")) : std::string("0ull");
    if(anyDelay || anyDynamics || anyPre || anyPost) { os << "#define GENNMI_DEVICE_MODULE 1      // the Makefile builds a gfx950 code object from this file as well" << std::endl; }
    modelMerged.genMergedSynapseDendriticDelayUpdateStructs(os, *this);
    modelMerged.genMergedPresynapticUpdateGroupStructs(os, *this);
    modelMerged.genMergedPostsynapticUpdateGroupStructs(os, *this);
    modelMerged.genMergedSynapseDynamicsGroupStructs(os, *this);
    for(const auto *k : {&delay, &dynamics, &pre, &post}) {
        if(k->table.numBlocks > 0) { k->args.define(os); }
    }
    os << std::endl;

    // ---- device pass
    os << "#ifdef __HIPCC__" << std::endl;
    os << "__device__ const gennmi_kernel::BlockEntry gennmiPresynapticBlocks[] = {" << std::endl << pre.table.entries.str() << "{0u, 0u, 0u, 0u}};" << std::endl;
    os << "__device__ const gennmi_kernel::BlockEntry gennmiPostsynapticBlocks[] = {" << std::endl << post.table.entries.str() << "{0u, 0u, 0u, 0u}};" << std::endl;
    os << "__device__ const gennmi_kernel::BlockEntry gennmiSynapseDynamicsBlocks[] = {" << std::endl << dynamics.table.entries.str() << "{0u, 0u, 0u, 0u}};" << std::endl;
    os << std::endl;
    if(anyDynamics) { dynamics.args.open(os, timeType); os << dynamics.body.str(); dynamics.args.close(os); }
    if(anyDelay) { delay.args.open(os, timeType, ""); os << delay.body.str(); delay.args.close(os); }
    if(anyPre) { pre.args.open(os, timeType); os << pre.body.str(); pre.args.close(os); }
    if(anyPost) { post.args.open(os, timeType); os << post.body.str(); post.args.close(os); }
    os << std::endl;

    // ---- host pass
    os << "#else" << std::endl;
    modelMerged.genMergedSynapseDendriticDelayUpdateHostStructArrayPush(os, *this);
    modelMerged.genMergedPresynapticUpdateGroupHostStructArrayPush(os, *this);
    modelMerged.genMergedPostsynapticUpdateGroupHostStructArrayPush(os, *this);
    modelMerged.genMergedSynapseDynamicsGroupHostStructArrayPush(os, *this);
    preambleHandler(os);
    for(const auto &g : modelMerged.getMergedSynapseDendriticDelayUpdateGroups()) { genDeviceStructArray(decl, upload, release, *this, g, "SynapseDendriticDelayUpdate", true); }
    for(const auto &g : modelMerged.getMergedPresynapticUpdateGroups()) { genDeviceStructArray(decl, upload, release, *this, g, "PresynapticUpdate"); }
    for(const auto &g : modelMerged.getMergedPostsynapticUpdateGroups()) { genDeviceStructArray(decl, upload, release, *this, g, "PostsynapticUpdate"); }
    for(const auto &g : modelMerged.getMergedSynapseDynamicsGroups()) { genDeviceStructArray(decl, upload, release, *this, g, "SynapseDynamics"); }
    os << declStream.str();
    os << "static bool gennmiSynapseLaunchesRegistered = false;" << std::endl;
    os << "extern \"C\" const unsigned char gennmi_synapseUpdate_image[];" << std::endl;
    os << "extern \"C\" const unsigned char gennmi_synapseUpdate_image_end[];" << std::endl;
    os << std::endl;
    os << "void gennmiUploadSynapseGroups()";
    {
        CodeStream::Scope b(os);
        os << uploadStream.str();
        // the first time: the launches of updateSynapses() in the order of the reference's function (backendCUDAHIP.cc:548-589):
        // ring pointers, synapse dynamics, presynaptic, postsynaptic; timers exist for the kinds of update the model has merged
        // groups of (generateRunner.cc:177-199)
        os << "if(!gennmiSynapseLaunchesRegistered)";
        {
            CodeStream::Scope b2(os);
            if(anyDelay || anyDynamics || anyPre || anyPost) {
                os << "uint32_t module = 0;" << std::endl;
                os << "GENNMI_CHECK(gennmi_program_load_module(gennmiProgram, gennmi_synapseUpdate_image, (size_t)(gennmi_synapseUpdate_image_end - gennmi_synapseUpdate_image), &module));" << std::endl;
            }
            if(anyDelay) {
                // The reference moves the ring pointers on at the start of every updateSynapses (backendCUDAHIP.cc:560-566), a launch
                // of one thread per group.  Here the last work-group of the neuron update to finish does it for the step that
                // follows (nothing reads the pointers in between), so the kernel below runs once, before the first step.
                CodeStream::Scope b3(os);
                os << "uint32_t k = 0;" << std::endl;
                os << "GENNMI_CHECK(gennmi_program_get_kernel(gennmiProgram, module, \"" << delay.args.name << "\", &k));" << std::endl;
                os << delay.args.fillBlock("nullptr", "0ull") << std::endl;
                os << "GENNMI_CHECK(gennmi_program_launch(gennmiProgram, k, 1u, 1u, 64u, &a, sizeof(a), 0.0, 0ull, -1));" << std::endl;
            }
            if(anyDynamics) { dynamics.args.addToPhase(os, "GENNMI_PHASE_SYNAPSES", dynamics.table.numBlocks, batchSize, 256, timing ? timerId("synapseDynamics") : -1, "nullptr", seed); }
            if(anyPre) { pre.args.addToPhase(os, "GENNMI_PHASE_SYNAPSES", pre.table.numBlocks, batchSize, 256, timing ? timerId("presynapticUpdate") : -1, "nullptr", seed); }
            if(anyPost) { post.args.addToPhase(os, "GENNMI_PHASE_SYNAPSES", post.table.numBlocks, batchSize, 256, timing ? timerId("postsynapticUpdate") : -1, "nullptr", seed); }
            os << "gennmiSynapseLaunchesRegistered = true;" << std::endl;
        }
    }
    os << std::endl;
    os << "void gennmiFreeSynapseGroups()";
    {
        CodeStream::Scope b(os);
        os << "gennmiSynapseLaunchesRegistered = false;" << std::endl;
        os << releaseStream.str();
    }
    os << std::endl;
    // (the generators' step counter — calls of updateSynapses so far — travels in the launch header)
    os << "void updateSynapses(" << model.getTimePrecision().getName() << " t)";
    {
        CodeStream::Scope b(os);
        os << "gennmiEnsureFinalised();" << std::endl;
        os << "GENNMI_CHECK(gennmi_program_update(gennmiProgram, GENNMI_PHASE_SYNAPSES, (double)t, 0u));" << std::endl;
    }
    os << "#endif" << std::endl;
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

    std::ostringstream declStream, uploadStream, releaseStream, deviceStream, hostStream, argsStream, lookupStream, kernelIdStream;
    CodeStream decl(declStream), upload(uploadStream), release(releaseStream), device(deviceStream), host(hostStream), argsDefs(argsStream), lookup(lookupStream);
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
        std::ostringstream neuronBody;
        KernelArgs neuronArgs("gennmiCustomUpdate" + name + "Kernel");
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
                    neuronArgs.add("MergedCustomUpdateGroup" + std::to_string(c.getIndex()), structArray);

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
        std::ostringstream wuBody, wuTables;
        KernelArgs wuArgs("gennmiCustomUpdateWU" + name + "Kernel");
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
                    wuArgs.add("MergedCustomUpdateWUGroup" + std::to_string(c.getIndex()), structArray);
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
        std::ostringstream trBody, trTables;
        KernelArgs trArgs("gennmiCustomUpdateTranspose" + name + "Kernel");
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
                    trArgs.add("MergedCustomUpdateTransposeWUGroup" + std::to_string(c.getIndex()), structArray);

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
        std::ostringstream ccBody, ccRemap;
        KernelArgs ccArgs("gennmiCustomConnectivityUpdate" + name + "Kernel");
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
                    ccArgs.add("MergedCustomConnectivityUpdateGroup" + std::to_string(c.getIndex()), structArray);
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
        const std::string seed = (model.getSeed() != 0) ? (std::to_string(model.getSeed()) + "ull") : std::string("gennmiRandomSeed()");
        // (a kernel's place in the program is looked up once, when the device copies of the struct arrays are first uploaded)
        auto declare = [&](const KernelArgs &k)
        {
            k.define(argsDefs);
            kernelIdStream << "static uint32_t " << k.name << "Id = 0;" << std::endl;
            lookup << "GENNMI_CHECK(gennmi_program_get_kernel(gennmiProgram, module, \"" << k.name << "\", &" << k.name << "Id));" << std::endl;
        };
        auto launch = [&](const KernelArgs &k, size_t gridX, size_t gridY, const std::string &seedExpr, const std::string &step, int timer)
        {
            CodeStream::Scope b(host);
            host << k.fillBlock("nullptr", seedExpr) << std::endl;
            host << "GENNMI_CHECK(gennmi_program_launch(gennmiProgram, " << k.name << "Id, " << gridX << "u, " << gridY << "u, 256u, &a, sizeof(a), (double)t, " << step << ", " << timer << "));" << std::endl;
        };
        if(neuronTable.numBlocks > 0) {
            declare(neuronArgs);
            device << "__device__ const gennmi_kernel::BlockEntry gennmiCustomUpdate" << name << "Blocks[] = {" << std::endl << neuronTable.entries.str() << "{0u, 0u, 0u, 0u}};" << std::endl;
            neuronArgs.open(device, timeType);
            device << neuronBody.str();
            neuronArgs.close(device);
        }
        if(wuBlocks > 0) {
            declare(wuArgs);
            device << wuTables.str();
            wuArgs.open(device, timeType);
            device << wuBody.str();
            wuArgs.close(device);
        }
        if(ccTable.numBlocks > 0) {
            declare(ccArgs);
            device << "__device__ const gennmi_kernel::BlockEntry gennmiCustomConnectivityUpdate" << name << "Blocks[] = {" << std::endl << ccTable.entries.str() << "{0u, 0u, 0u, 0u}};" << std::endl;
            ccArgs.open(device, timeType);
            device << ccBody.str();
            ccArgs.close(device);
        }
        if(trBlocks > 0) {
            declare(trArgs);
            device << trTables.str();
            trArgs.open(device, timeType);
            device << "__shared__ " << model.getPrecision().getName() << " gennmiTile[64][65];" << std::endl;
            device << trBody.str();
            trArgs.close(device);
        }
        host << "void update" << name << "(unsigned long long timestep)";
        {
            CodeStream::Scope b(host);
            host << "gennmiEnsureFinalised();" << std::endl;
            // (every launch below first runs the steps still noted — the library's queue and the program's — and goes to the
            // stream the step's kernels use)
            host << "const " << timeType << " t = timestep * " << Type::writeNumeric(model.getDT(), model.getTimePrecision()) << ";" << std::endl;
            const bool timing = model.isTimingEnabled();
            const int timer = timing ? timerId("customUpdate" + name) : -1, transposeTimer = timing ? timerId("customUpdate" + name + "Transpose") : -1;
            host << ccHost.str();
            if(ccTable.numBlocks > 0) {
                // (connectivity first, like the reference: single_threaded_cpu/backend.cc:824-860; the generator's step counts this group's calls)
                host << "static unsigned long long gennmiCalls = 0;" << std::endl;
                launch(ccArgs, ccTable.numBlocks, 1, seed, "gennmiCalls++", timer);
                host << ccRemap.str();
            }
            if(neuronTable.numBlocks > 0) { launch(neuronArgs, neuronTable.numBlocks, batchSize, "0ull", "0ull", timer); }
            if(wuBlocks > 0) { launch(wuArgs, wuBlocks, batchSize, "0ull", "0ull", timer); }
            if(trBlocks > 0) { launch(trArgs, trBlocks, batchSize, "0ull", "0ull", transposeTimer); }
            host << notes.str();
            if(timing) {
                // (these counters are not part of stepTime: read here, after the group's kernels have finished, backendCUDAHIP.cc:826-856)
                host << "GENNMI_CHECK(gennmi_program_get_time(gennmiProgram, " << timer << ", &customUpdate" << name << "Time));" << std::endl;
                host << "GENNMI_CHECK(gennmi_program_get_time(gennmiProgram, " << transposeTimer << ", &customUpdate" << name << "TransposeTime));" << std::endl;
            }
        }
        host << std::endl;
    }

    // struct definitions (both passes), then the kernels (device pass) or the host arrays, push functions and update functions (host pass)
    if(!deviceStream.str().empty()) { os << "#define GENNMI_DEVICE_MODULE 1      // the Makefile builds a gfx950 code object from this file as well" << std::endl; }
    modelMerged.genMergedCustomUpdateStructs(os, *this);
    modelMerged.genMergedCustomUpdateWUStructs(os, *this);
    modelMerged.genMergedCustomUpdateTransposeWUStructs(os, *this);
    modelMerged.genMergedCustomConnectivityUpdateStructs(os, *this);
    modelMerged.genMergedCustomConnectivityRemapUpdateStructs(os, *this);
    modelMerged.genMergedCustomConnectivityHostUpdateStructs(os, *this);
    os << argsStream.str();
    os << std::endl;
    os << "#ifdef __HIPCC__" << std::endl;
    os << deviceStream.str();
    os << "#else" << std::endl;
    modelMerged.genMergedCustomConnectivityHostUpdateStructArrayPush(os, *this);
    modelMerged.genMergedCustomConnectivityUpdateHostStructArrayPush(os, *this);
    modelMerged.genMergedCustomConnectivityRemapUpdateHostStructArrayPush(os, *this);
    modelMerged.genMergedCustomUpdateHostStructArrayPush(os, *this);
    modelMerged.genMergedCustomUpdateWUHostStructArrayPush(os, *this);
    modelMerged.genMergedCustomUpdateTransposeWUHostStructArrayPush(os, *this);
    preambleHandler(os);
    for(const auto &g : modelMerged.getMergedCustomUpdateGroups()) { genDeviceStructArray(decl, upload, release, *this, g, "CustomUpdate"); }
    for(const auto &g : modelMerged.getMergedCustomUpdateWUGroups()) { genDeviceStructArray(decl, upload, release, *this, g, "CustomUpdateWU"); }
    for(const auto &g : modelMerged.getMergedCustomUpdateTransposeWUGroups()) { genDeviceStructArray(decl, upload, release, *this, g, "CustomUpdateTransposeWU"); }
    for(const auto &g : modelMerged.getMergedCustomConnectivityUpdateGroups()) { genDeviceStructArray(decl, upload, release, *this, g, "CustomConnectivityUpdate"); }
    os << declStream.str();
    os << kernelIdStream.str();
    os << "static bool gennmiCustomUpdateKernelsLoaded = false;" << std::endl;
    os << "extern \"C\" const unsigned char gennmi_customUpdate_image[];" << std::endl;
    os << "extern \"C\" const unsigned char gennmi_customUpdate_image_end[];" << std::endl;
    os << std::endl;
    os << "void gennmiUploadCustomUpdateGroups()";
    {
        CodeStream::Scope b(os);
        os << uploadStream.str();
        if(!lookupStream.str().empty()) {
            os << "if(!gennmiCustomUpdateKernelsLoaded)";
            CodeStream::Scope b2(os);
            os << "uint32_t module = 0;" << std::endl;
            os << "GENNMI_CHECK(gennmi_program_load_module(gennmiProgram, gennmi_customUpdate_image, (size_t)(gennmi_customUpdate_image_end - gennmi_customUpdate_image), &module));" << std::endl;
            os << lookupStream.str();
            os << "gennmiCustomUpdateKernelsLoaded = true;" << std::endl;
        }
    }
    os << std::endl;
    os << "void gennmiFreeCustomUpdateGroups()";
    {
        CodeStream::Scope b(os);
        os << "gennmiCustomUpdateKernelsLoaded = false;" << std::endl;
        os << releaseStream.str();
    }
    os << std::endl;
    os << hostStream.str();
    os << "#endif" << std::endl;
}
}   // namespace GeNN::CodeGenerator::MI355X
