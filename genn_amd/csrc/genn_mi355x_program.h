// Programs: generated gfx950 code objects loaded and launched behind the C ABI (included by genn_mi355x.hip).
//
// The reference's generated runner launches its kernels inline (`kernel<<<grid, block>>>(...)`,
// src/genn/genn/code_generator/backendCUDAHIP.cc:386-420, 548-589, 750-856) and so has to be compiled by the device
// compiler.  Here the runner is host C++: the device code of a model is a code object per module, and everything that
// touches HIP — module loading, launches, the stream, timer events, graph capture, the error flag — is in this file.
//
// Step values (time, recording row, random-number step, look-back tag) reach a kernel through the launch header
// (gennmi_launch_header_t): by value for a launch made when asked for, or as an index into a device table for launches
// replayed from a captured graph, whose kernel arguments are fixed at capture.  The table is refilled with one
// stream-ordered copy from pinned memory before every replay.
#pragma once

struct gennmi_program
{
    gennmi_runner *runner = nullptr;
    hipStream_t stream = nullptr; bool ownStream = false;
    std::vector<hipModule_t> modules;
    std::vector<hipFunction_t> kernels;
    struct Launch { uint32_t kernel, gridX, gridY, blockX; int timer; std::vector<unsigned char> args; };
    std::vector<Launch> phases[GENNMI_NUM_PHASES];
    unsigned long long phaseCalls[GENNMI_NUM_PHASES] = {0, 0};
    uint32_t phaseTag[GENNMI_NUM_PHASES] = {0, 0};
    uint32_t spinLimit = 1u << 22;
    uint32_t *dError = nullptr, *hError = nullptr;
    bool flagCopyPending = false;       // launches were made since the flag was last copied to hError
    // queue of noted calls
    struct Call { int phase; double t; uint32_t recordingTimestep; };
    uint32_t queueLimit = 0;            // in calls
    std::vector<Call> queued;
    // graph of a full queue
    gennmi_step_entry_t *dTable = nullptr;
    static constexpr int STAGES = 4;
    gennmi_step_entry_t *hTable[STAGES] = {nullptr, nullptr, nullptr, nullptr};
    hipEvent_t stageFree[STAGES] = {nullptr, nullptr, nullptr, nullptr};
    bool stageUsed[STAGES] = {false, false, false, false};
    int nextStage = 0;
    hipGraphExec_t graphExec = nullptr;
    std::vector<int> graphPattern;
    // timers
    bool timing = false;
    double seconds[GENNMI_MAX_TIMERS] = {};
    struct Pending { hipEvent_t a, b; int timer; };
    std::vector<hipEvent_t> eventPool; size_t eventNext = 0; std::vector<Pending> pending;
    // statistics
    unsigned long long callsExecuted = 0, callsReplayed = 0, launchesMade = 0, graphsCaptured = 0;
};

static std::vector<gennmi_program*> g_programs;             // guarded by g_runnersMutex
static std::atomic<int> g_programsPending{0};               // programs with noted calls or an error flag not yet copied

static void programNotePending(gennmi_program *p, bool &was)
{
    if(!was) { was = true; g_programsPending++; }
    (void)p;
}
static bool programIsPending(const gennmi_program *p) { return !p->queued.empty() || p->flagCopyPending; }

static int programLaunch(gennmi_program *p, const gennmi_program::Launch &l, const gennmi_launch_header_t &header)
{
    alignas(16) unsigned char buffer[sizeof(gennmi_launch_header_t) + GENNMI_MAX_LAUNCH_ARG_BYTES];
    static_assert(sizeof(gennmi_launch_header_t) % 8 == 0, "the launch's own arguments follow the header 8-byte aligned");
    memcpy(buffer, &header, sizeof(header));
    if(!l.args.empty()) { memcpy(buffer + sizeof(header), l.args.data(), l.args.size()); }
    size_t size = sizeof(header) + l.args.size();
    void *config[] = {HIP_LAUNCH_PARAM_BUFFER_POINTER, buffer, HIP_LAUNCH_PARAM_BUFFER_SIZE, &size, HIP_LAUNCH_PARAM_END};
    hipEvent_t e0 = nullptr, e1 = nullptr;
    const bool timed = p->timing && l.timer >= 0;
    auto stampEvent = [p](hipEvent_t *out) -> int {
        if(p->eventNext == p->eventPool.size()) { hipEvent_t e; HIP_TRY(hipEventCreate(&e)); p->eventPool.push_back(e); }
        *out = p->eventPool[p->eventNext++];
        HIP_TRY(hipEventRecord(*out, p->stream));
        return GENNMI_OK;
    };
    if(timed) { const int rc = stampEvent(&e0); if(rc) { return rc; } }
    HIP_TRY(hipModuleLaunchKernel(p->kernels[l.kernel], l.gridX, l.gridY, 1, l.blockX, 1, 1, 0, p->stream, nullptr, config));
    if(timed) { const int rc = stampEvent(&e1); if(rc) { return rc; } p->pending.push_back({e0, e1, l.timer}); }
    p->launchesMade++;
    return GENNMI_OK;
}

static int programDrainTimers(gennmi_program *p)
{
    if(p->pending.empty()) { return GENNMI_OK; }
    HIP_TRY(hipStreamSynchronize(p->stream));
    for(const auto &e : p->pending) {
        float ms = 0;
        HIP_TRY(hipEventElapsedTime(&ms, e.a, e.b));
        p->seconds[e.timer] += ms * 1e-3;
    }
    p->pending.clear();
    p->eventNext = 0;
    return GENNMI_OK;
}

static gennmi_step_entry_t programEntry(gennmi_program *p, const gennmi_program::Call &c)
{
    gennmi_step_entry_t e;
    e.t = c.t;
    e.step = p->phaseCalls[c.phase]++;
    e.recordingTimestep = c.recordingTimestep;
    p->phaseTag[c.phase] = (p->phaseTag[c.phase] == 0xFFFFFFFFu) ? 1u : p->phaseTag[c.phase] + 1u;
    e.tag = p->phaseTag[c.phase];
    return e;
}

// one call of a phase, launched now
static int programRunCall(gennmi_program *p, const gennmi_program::Call &c)
{
    gennmi_launch_header_t header{};
    header.steps = nullptr; header.k = 0; header.spinLimit = p->spinLimit;
    header.inlineEntry = programEntry(p, c);
    for(const auto &l : p->phases[c.phase]) {
        if(p->timing && p->pending.size() >= 2048) { const int rc = programDrainTimers(p); if(rc) { return rc; } }
        const int rc = programLaunch(p, l, header);
        if(rc) { return rc; }
    }
    p->callsExecuted++;
    return GENNMI_OK;
}

// Executes the noted calls: a full queue whose phases come in the order of the captured graph (or of no graph yet) is
// replayed from the graph, anything else is launched call by call.  On failure the calls not yet executed stay noted.
static int flushProgram(gennmi_program *p)
{
    bool wasPending = programIsPending(p);
    if(!p->queued.empty()) {
        std::vector<gennmi_program::Call> calls;
        calls.swap(p->queued);
        bool replay = (p->queueLimit != 0 && calls.size() == p->queueLimit && !p->timing);
        if(replay && p->graphExec) {
            for(size_t i = 0; i < calls.size() && replay; i++) { replay = (calls[i].phase == p->graphPattern[i]); }
        }
        size_t done = 0;
        int rc = GENNMI_OK;
        auto giveBack = [&]() { p->queued.insert(p->queued.begin(), calls.begin() + done, calls.end()); };
        if(replay) {
            const int stage = p->nextStage;
            p->nextStage = (p->nextStage + 1) % gennmi_program::STAGES;
            if(p->stageUsed[stage]) { HIP_TRY(hipEventSynchronize(p->stageFree[stage])); }
            if(!p->graphExec) {
                hipGraph_t graph;
                HIP_TRY(hipStreamBeginCapture(p->stream, hipStreamCaptureModeThreadLocal));
                for(size_t i = 0; i < calls.size() && rc == GENNMI_OK; i++) {
                    gennmi_launch_header_t header{};
                    header.steps = p->dTable; header.k = (uint32_t)i; header.spinLimit = p->spinLimit;
                    for(const auto &l : p->phases[calls[i].phase]) {
                        rc = programLaunch(p, l, header);
                        if(rc) { break; }
                    }
                }
                const hipError_t ce = hipStreamEndCapture(p->stream, &graph);
                if(rc) { giveBack(); return rc; }
                if(ce != hipSuccess) { giveBack(); return fail(GENNMI_EHIP, std::string("hipStreamEndCapture: ") + hipGetErrorString(ce)); }
                const hipError_t ie = hipGraphInstantiate(&p->graphExec, graph, nullptr, nullptr, 0);
                hipGraphDestroy(graph);
                if(ie != hipSuccess) { p->graphExec = nullptr; giveBack(); return fail(GENNMI_EHIP, std::string("hipGraphInstantiate: ") + hipGetErrorString(ie)); }
                p->graphPattern.resize(calls.size());
                for(size_t i = 0; i < calls.size(); i++) { p->graphPattern[i] = calls[i].phase; }
                p->graphsCaptured++;
            }
            for(size_t i = 0; i < calls.size(); i++) { p->hTable[stage][i] = programEntry(p, calls[i]); }
            HIP_TRY(hipMemcpyAsync(p->dTable, p->hTable[stage], calls.size() * sizeof(gennmi_step_entry_t), hipMemcpyHostToDevice, p->stream));
            HIP_TRY(hipEventRecord(p->stageFree[stage], p->stream));
            p->stageUsed[stage] = true;
            HIP_TRY(hipGraphLaunch(p->graphExec, p->stream));
            p->callsExecuted += calls.size();
            p->callsReplayed += calls.size();
            done = calls.size();
        }
        else {
            for(; done < calls.size(); done++) {
                rc = programRunCall(p, calls[done]);
                if(rc) { giveBack(); return rc; }
            }
        }
        p->flagCopyPending = true;
    }
    if(p->flagCopyPending) {
        // the flag travels on the stream behind the work, so that whoever waits for the work next finds it in host memory
        HIP_TRY(hipMemcpyAsync(p->hError, p->dError, sizeof(uint32_t), hipMemcpyDeviceToHost, p->stream));
        p->flagCopyPending = false;
    }
    if(wasPending && !programIsPending(p)) { g_programsPending--; }
    return GENNMI_OK;
}

static int flushPrograms()
{
    if(g_programsPending.load(std::memory_order_relaxed) == 0) { return GENNMI_OK; }
    std::vector<gennmi_program*> programs;
    {
        std::lock_guard<std::mutex> lock(g_runnersMutex);
        programs = g_programs;
    }
    for(gennmi_program *p : programs) {
        const int rc = flushProgram(p);
        if(rc) { return rc; }
    }
    return GENNMI_OK;
}

// after a wait that covered every program's stream: has a kernel raised its program's error flag?
static int checkPrograms()
{
    std::lock_guard<std::mutex> lock(g_runnersMutex);
    for(const gennmi_program *p : g_programs) {
        if(*p->hError) {
            return fail(GENNMI_EDEVICE, "a generated kernel's bounded wait for other work-groups expired (spike-queue offsets); state is undefined");
        }
    }
    return GENNMI_OK;
}

extern "C" {

int gennmi_program_create(gennmi_program **program, gennmi_runner *runner, uint32_t stepQueueLength)
{
    if(!program) { return fail(GENNMI_EINVAL, "program_create: null argument"); }
    if(stepQueueLength > 4096) { return fail(GENNMI_EINVAL, "program_create: at most 4096 queued steps"); }
    gennmi_program *p = new gennmi_program;
    p->runner = runner;
    if(runner) { p->stream = runner->stream; }
    else { HIP_TRY(hipStreamCreate(&p->stream)); p->ownStream = true; }      // blocking stream: ordered against null-stream copies
    HIP_TRY(hipMalloc(&p->dError, sizeof(uint32_t)));
    HIP_TRY(hipMemset(p->dError, 0, sizeof(uint32_t)));
    HIP_TRY(hipHostMalloc(reinterpret_cast<void**>(&p->hError), sizeof(uint32_t), hipHostMallocDefault));
    *p->hError = 0;
    p->queueLimit = stepQueueLength * GENNMI_NUM_PHASES;
    if(p->queueLimit) {
        HIP_TRY(hipMalloc(&p->dTable, p->queueLimit * sizeof(gennmi_step_entry_t)));
        for(int s = 0; s < gennmi_program::STAGES; s++) {
            HIP_TRY(hipHostMalloc(reinterpret_cast<void**>(&p->hTable[s]), p->queueLimit * sizeof(gennmi_step_entry_t), hipHostMallocDefault));
            HIP_TRY(hipEventCreateWithFlags(&p->stageFree[s], hipEventDisableTiming));
        }
    }
    if(const char *envSpin = getenv("GENNMI_SPIN_LIMIT")) { p->spinLimit = (uint32_t)std::max(0ll, atoll(envSpin)); }
    {
        std::lock_guard<std::mutex> lock(g_runnersMutex);
        g_programs.push_back(p);
    }
    *program = p;
    return GENNMI_OK;
}

int gennmi_program_destroy(gennmi_program *p)
{
    if(!p) { return GENNMI_OK; }
    if(programIsPending(p)) { p->queued.clear(); p->flagCopyPending = false; g_programsPending--; }      // nothing can observe these calls any more
    {
        std::lock_guard<std::mutex> lock(g_runnersMutex);
        g_programs.erase(std::remove(g_programs.begin(), g_programs.end(), p), g_programs.end());
    }
    hipStreamSynchronize(p->stream);
    if(getenv("GENNMI_PROGRAM_STATS")) {
        fprintf(stderr, "gennmi_program: calls %llu, replayed %llu, launches %llu, graphs %llu\n", p->callsExecuted, p->callsReplayed, p->launchesMade, p->graphsCaptured);
    }
    if(p->graphExec) { hipGraphExecDestroy(p->graphExec); }
    for(hipEvent_t e : p->eventPool) { hipEventDestroy(e); }
    for(int s = 0; s < gennmi_program::STAGES; s++) {
        if(p->hTable[s]) { hipHostFree(p->hTable[s]); }
        if(p->stageFree[s]) { hipEventDestroy(p->stageFree[s]); }
    }
    hipFree(p->dTable); hipFree(p->dError);
    if(p->hError) { hipHostFree(p->hError); }
    for(hipModule_t m : p->modules) { hipModuleUnload(m); }
    if(p->ownStream) { hipStreamDestroy(p->stream); }
    delete p;
    return GENNMI_OK;
}

int gennmi_program_load_module(gennmi_program *p, const void *image, size_t bytes, uint32_t *module)
{
    if(!p || !image || bytes == 0 || !module) { return fail(GENNMI_EINVAL, "program_load_module: bad arguments"); }
    hipModule_t m;
    HIP_TRY(hipModuleLoadData(&m, image));
    p->modules.push_back(m);
    *module = (uint32_t)(p->modules.size() - 1);
    return GENNMI_OK;
}

int gennmi_program_get_kernel(gennmi_program *p, uint32_t module, const char *name, uint32_t *kernel)
{
    if(!p || !name || !kernel || module >= p->modules.size()) { return fail(GENNMI_EINVAL, "program_get_kernel: bad arguments"); }
    hipFunction_t f;
    const hipError_t e = hipModuleGetFunction(&f, p->modules[module], name);
    if(e != hipSuccess) { return fail(GENNMI_EHIP, std::string("program_get_kernel: no kernel '") + name + "' in the module: " + hipGetErrorString(e)); }
    p->kernels.push_back(f);
    *kernel = (uint32_t)(p->kernels.size() - 1);
    return GENNMI_OK;
}

int gennmi_program_error_flag(gennmi_program *p, uint32_t **deviceFlag)
{
    if(!p || !deviceFlag) { return fail(GENNMI_EINVAL, "program_error_flag: null argument"); }
    *deviceFlag = p->dError;
    return GENNMI_OK;
}

static int programCheckLaunch(const gennmi_program *p, const char *who, uint32_t kernel, uint32_t gridX, uint32_t gridY, uint32_t blockX,
                              const void *args, size_t argBytes, int timer)
{
    if(!p || kernel >= p->kernels.size()) { return fail(GENNMI_EINVAL, std::string(who) + ": no such kernel"); }
    if(gridX == 0 || gridY == 0 || gridY > 65535 || blockX == 0 || blockX > 1024) { return fail(GENNMI_EINVAL, std::string(who) + ": bad launch dimensions"); }
    if((argBytes && !args) || argBytes > GENNMI_MAX_LAUNCH_ARG_BYTES || (argBytes % 8) != 0) { return fail(GENNMI_EINVAL, std::string(who) + ": argument block must be a multiple of 8 bytes, at most GENNMI_MAX_LAUNCH_ARG_BYTES"); }
    if(timer < -1 || timer >= GENNMI_MAX_TIMERS) { return fail(GENNMI_EINVAL, std::string(who) + ": no such timer"); }
    return GENNMI_OK;
}

int gennmi_program_add_launch(gennmi_program *p, int phase, uint32_t kernel, uint32_t gridX, uint32_t gridY, uint32_t blockX,
                              const void *args, size_t argBytes, int timer)
{
    { const int rc = programCheckLaunch(p, "program_add_launch", kernel, gridX, gridY, blockX, args, argBytes, timer); if(rc) { return rc; } }
    if(phase < 0 || phase >= GENNMI_NUM_PHASES) { return fail(GENNMI_EINVAL, "program_add_launch: no such phase"); }
    { const int rc = flushProgram(p); if(rc) { return rc; } }
    if(p->graphExec) { HIP_TRY(hipStreamSynchronize(p->stream)); hipGraphExecDestroy(p->graphExec); p->graphExec = nullptr; }
    gennmi_program::Launch l{kernel, gridX, gridY, blockX, timer, {}};
    l.args.assign(static_cast<const unsigned char*>(args), static_cast<const unsigned char*>(args) + argBytes);
    p->phases[phase].push_back(std::move(l));
    return GENNMI_OK;
}

int gennmi_program_clear_phases(gennmi_program *p)
{
    if(!p) { return fail(GENNMI_EINVAL, "program_clear_phases: null program"); }
    { const int rc = flushProgram(p); if(rc) { return rc; } }
    if(p->graphExec) { HIP_TRY(hipStreamSynchronize(p->stream)); hipGraphExecDestroy(p->graphExec); p->graphExec = nullptr; }
    for(auto &ph : p->phases) { ph.clear(); }
    return GENNMI_OK;
}

int gennmi_program_update(gennmi_program *p, int phase, double t, uint32_t recordingTimestep)
{
    if(!p || phase < 0 || phase >= GENNMI_NUM_PHASES) { return fail(GENNMI_EINVAL, "program_update: bad arguments"); }
    const gennmi_program::Call call{phase, t, recordingTimestep};
    if(p->queueLimit && !p->timing) {
        bool was = programIsPending(p);
        p->queued.push_back(call);
        programNotePending(p, was);
        return (p->queued.size() >= p->queueLimit) ? flushProgram(p) : GENNMI_OK;
    }
    FLUSH_QUEUED();
    const int rc = programRunCall(p, call);
    if(rc) { return rc; }
    bool was = programIsPending(p);
    p->flagCopyPending = true;
    programNotePending(p, was);
    return GENNMI_OK;
}

int gennmi_program_launch(gennmi_program *p, uint32_t kernel, uint32_t gridX, uint32_t gridY, uint32_t blockX,
                          const void *args, size_t argBytes, double t, unsigned long long step, int timer)
{
    { const int rc = programCheckLaunch(p, "program_launch", kernel, gridX, gridY, blockX, args, argBytes, timer); if(rc) { return rc; } }
    FLUSH_QUEUED();
    gennmi_program::Launch l{kernel, gridX, gridY, blockX, timer, {}};
    l.args.assign(static_cast<const unsigned char*>(args), static_cast<const unsigned char*>(args) + argBytes);
    gennmi_launch_header_t header{};
    header.steps = nullptr; header.k = 0; header.spinLimit = p->spinLimit;
    header.inlineEntry.t = t; header.inlineEntry.step = step; header.inlineEntry.recordingTimestep = 0; header.inlineEntry.tag = 1;
    const int rc = programLaunch(p, l, header);
    if(rc) { return rc; }
    bool was = programIsPending(p);
    p->flagCopyPending = true;
    programNotePending(p, was);
    return GENNMI_OK;
}

int gennmi_program_synchronize(gennmi_program *p)
{
    if(!p) { return fail(GENNMI_EINVAL, "program_synchronize: null program"); }
    FLUSH_QUEUED();
    HIP_TRY(hipStreamSynchronize(p->stream));
    if(*p->hError) { return fail(GENNMI_EDEVICE, "a generated kernel's bounded wait for other work-groups expired (spike-queue offsets); state is undefined"); }
    return GENNMI_OK;
}

int gennmi_program_set_timing(gennmi_program *p, int enabled)
{
    if(!p) { return fail(GENNMI_EINVAL, "program_set_timing: null program"); }
    FLUSH_QUEUED();
    if(!enabled) { const int rc = programDrainTimers(p); if(rc) { return rc; } }
    p->timing = (enabled != 0);
    return GENNMI_OK;
}

int gennmi_program_get_time(gennmi_program *p, int timer, double *seconds)
{
    if(!p || !seconds || timer < 0 || timer >= GENNMI_MAX_TIMERS) { return fail(GENNMI_EINVAL, "program_get_time: bad arguments"); }
    FLUSH_QUEUED();
    { const int rc = programDrainTimers(p); if(rc) { return rc; } }
    *seconds = p->seconds[timer];
    return GENNMI_OK;
}

int gennmi_program_get_info(gennmi_program *p, unsigned long long info[4])
{
    if(!p || !info) { return fail(GENNMI_EINVAL, "program_get_info: null argument"); }
    FLUSH_QUEUED();
    info[0] = p->callsExecuted; info[1] = p->callsReplayed; info[2] = p->launchesMade; info[3] = p->graphsCaptured;
    return GENNMI_OK;
}

}   // extern "C"
