// MI355X (gfx950) device layer for GeNN's per-timestep hot path: kernels + C ABI.
//
// This file holds the runner (launch plans, graph capture, the C entry points); the kernels live in the headers it
// includes: genn_mi355x_device.h (descriptor tables, helpers), genn_mi355x_synapse_kernels.h, genn_mi355x_neuron_kernels.h,
// genn_mi355x_resident_kernels.h.
//
// Kernels (one launch each per timestep, all on the runner's stream):
//   presynapticUpdateKernel   sparse / Toeplitz presynaptic event propagation into outPost or the
//                             dendritic-delay ring (replaces updatePresynapticKernel,
//                             src/genn/genn/code_generator/backendSIMT.cc:694-764 and the strategies in
//                             presynapticUpdateStrategySIMT.cc:57-162, 167-389, 750-934)
//   postsynapticUpdateKernel  STDP learnPost through the column remap (backendSIMT.cc:766-803, 1822-1898)
//   neuronUpdateKernel        PSM apply + current sources + neuron model + threshold + ordered spike
//                             compaction + recording (backendSIMT.cc:405-662, 1931-1975); also does the
//                             work of neuronSpikeQueueUpdateKernel (:373-403) and
//                             synapseDendriticDelayUpdateKernel (:664-692), which need no launch here.
//   residentKernel            many timesteps of a network that fits the chip in ONE launch: neuron state in registers,
//                             inSyn and dendritic-delay rings in LDS, spikes exchanged between work-groups through
//                             one word per tile (no counterpart in the reference)
//   remap*Kernel              deterministic colLength/remap build (replaces backendSIMT.cc:1977-1991)
//
// Arithmetic contract: fp32, one rounding per operation, same operation order as the code the
// reference's SingleThreadedCPU backend generates (build with -ffp-contract=off).  The only
// permitted divergence is the order of fp32 atomic adds into outPost / denDelay.
#include <dlfcn.h>
#include <sys/mman.h>
#include <hip/hip_runtime.h>

#include <algorithm>
#include <atomic>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <type_traits>
#include <map>
#include <mutex>
#include <chrono>
#include <vector>

#include "genn_mi355x.h"
#include "genn_mi355x_rows.h"

// device-side tables, constants and helpers; the synapse, neuron and resident-plan kernels
#include "genn_mi355x_device.h"
#include "genn_mi355x_synapse_kernels.h"
#include "genn_mi355x_neuron_kernels.h"
#include "genn_mi355x_resident_kernels.h"
#include "genn_mi355x_ordered_kernels.h"
#include "genn_mi355x_conv_step_kernels.h"

struct gennmi_runner
{
    float dt = 0;
    uint32_t batch = 1;
    bool finalised = false;
    hipStream_t stream = nullptr;
    std::vector<NeuronGroupDev> neuron; std::vector<PreGroupDev> pre; std::vector<PostGroupDev> post;
    std::vector<DenseGroupDev> dense; DenseGroupDev *dDense = nullptr; uint32_t denseBlocks = 0;
    std::vector<ProcGroupDev> proc; ProcGroupDev *dProc = nullptr; uint32_t procBlocks = 0;
    NeuronGroupDev *dNeuron = nullptr; PreGroupDev *dPre = nullptr; PostGroupDev *dPost = nullptr;
    uint32_t neuronBlocks = 0, preBlocks = 0, postBlocks = 0;
    unsigned long long *dAgg = nullptr; uint32_t *dError = nullptr; unsigned long long *dEvents = nullptr;
    uint32_t *hError = nullptr;     // the error flag: a pinned host word; dError is the same word's device address
    StepState *dState = nullptr;
    unsigned long long epoch = 0;       // completed steps (host mirror)
    bool synapsesDone = false;          // updateSynapses ran for the current step
    bool fusedStep = false;             // zero-delay synapses are delivered by the neuron update; one launch per step
    TileGroupDev *dTile = nullptr; uint32_t tileBlocks = 0, tileFloats = 0, tileThreads = BLOCK;
    uint32_t postLdsBytes = 0;
    // one launch for the scatter path, the tile path and the paired postsynaptic passes of a step (synapseCombinedKernel)
    bool combineSynapses = false, combinePost = false; uint32_t synapseThreads = BLOCK; size_t combinedLdsBytes = 0;
    ConvTileDev *dConvTile = nullptr; uint32_t convTileBlocks = 0; size_t convTileBytes = 0;
    ConvMfmaDev *dConvMfma = nullptr; uint32_t convMfmaBlocks = 0; size_t convMfmaBytes = 0;      // Conv2D on the matrix cores (instead of dConvTile)
    ConvMfmaDev convMfma{}; size_t convSource = 0;      // host copy of its descriptor; index of its source population in `neuron`
    // a convolutional layer's whole step in one launch (convStepKernel): the layer's target population is updated on the accumulators
    bool convStep = false;
    NeuronGroupDev *dConvTarget = nullptr, *dConvRest = nullptr; uint32_t convRestBlocks = 0; size_t convStepBytes = 0;
    unsigned long long *dConvAgg = nullptr, *dConvRestAgg = nullptr;
    bool bitmapsStale = false;          // a spike queue was written by the caller: the bitmaps kept beside the queues are rebuilt before the next step
    std::vector<void*> owned;           // engine-private device allocations (shadow queues, zero-delay lists)
    // resident plan (many steps per launch)
    bool resident = false;
    ResTile *dResTiles = nullptr; NeuronGroupDev *dResGroups = nullptr; uint8_t *dResTileGroup = nullptr;
    unsigned long long *dResTags = nullptr, *dResSide = nullptr;
    uint32_t resTiles = 0, resReplicaStride = 0; unsigned long long resSeq = 0; size_t resLdsBytes = 0; bool resPoisson = false;
    std::vector<u32x4*> resSegs;        // segment table of each presynaptic group, in push order
    std::vector<uint32_t> resSegTiles;  // tiles of its target population
    std::vector<u32x2*> resPacked;      // its synapses as the resident kernel reads them
    uint32_t neuronsPerLane = 1;        // 2, 4 or 8: neuronBulkKernel instead of neuronUpdateKernel
    bool plainGroups = false;           // every group is one the several-neurons-per-lane neuron update covers
    bool sourcesStale = false;          // startSpike / endSpike / spikeTimes of a spike source were written since nextSpikeTime was built
    bool failed = false;                // a queued step failed part-way: what was queued behind it is lost, the runner refuses to go on
    bool resStale = false;              // connectivity or weights were written since the tables were built ...
    std::vector<uint8_t> resStaleProj;  // ... of these projections (index into pre)
    bool tablesStale = false;           // rowLength / ind / d of a projection were written since the connectivity-derived tables were built
    // connectivity-derived tables that are rebuilt when tablesStale: segment boundaries of the tile path ...
    struct TileTable { size_t pre; uint16_t *off; uint32_t tileSize, numTiles; };
    std::vector<TileTable> tileTables;
    // segment records of the tile path (copies of static weights and targets, one aligned record per (row, tile)): rebuilt
    // when the projection's connectivity or weights have been written
    struct RecordTable { size_t pre; uint8_t *records; uint8_t *overflow; const uint16_t *off; uint32_t lanes, tileSize, numTiles; };
    std::vector<RecordTable> recordTables;
    bool recordsStale = false;
    std::vector<void*> zeroOwned;       // ... the zero-delay lists of the single-launch step ...
    // ... and the column views of ordered accumulation (validation mode: every element summed in the CPU backend's order)
    bool ordered = false;
    std::vector<OrderedGroupDev> orderedGroups; std::vector<size_t> orderedPre;
    std::vector<OrderedSourceDev> orderedSources; OrderedSourceDev *dOrderedSources = nullptr; uint32_t orderedSourceBlocks = 0;
    uint32_t *dOrderedBitmaps = nullptr; size_t orderedBitmapWords = 0;
    std::vector<void*> orderedOwned;
    bool scatterNeeded = true;          // some presynaptic group still goes through presynapticUpdateKernel
    // graph
    hipGraphExec_t graphExec = nullptr; unsigned long long graphSteps = 0;
    // timing
    bool timing = false;
    double neuronTime = 0, preTime = 0, postTime = 0;
    unsigned long long preLaunches = 0, neuronLaunches = 0, postLaunches = 0, stepLaunches = 0;
    double stepTime = 0;                // single-launch steps
    struct Pending { hipEvent_t a, b; int kind; };          // kind: 0 presynaptic, 1 postsynaptic, 2 neuron, 3 single-launch step
    std::vector<hipEvent_t> eventPool; size_t eventNext = 0; std::vector<Pending> pending;
    hipEvent_t marks[2] = {nullptr, nullptr};               // gennmi_runner_stream_mark
    // step queue (gennmi_runner_set_step_queue): steps asked for one at a time and not yet launched
    struct QueuedStep { float t; uint32_t recordingTimestep; };
    uint32_t stepQueueLimit = 0;
    std::vector<QueuedStep> queued;
};

// Runners whose resident plan holds copies of weights (inline in the segment tables): a write to device memory that
// overlaps one of their projections' arrays makes them rebuild the tables before the next resident launch.
static std::mutex g_runnersMutex;
static std::vector<gennmi_runner*> g_runners;

static void noteDeviceWrite(const void *dev, size_t bytes)
{
    std::lock_guard<std::mutex> lock(g_runnersMutex);
    const uintptr_t a = reinterpret_cast<uintptr_t>(dev), b = a + bytes;
    for(gennmi_runner *r : g_runners) {
        for(const auto &n : r->neuron) {
            if(n.spikeBitmap && !r->bitmapsStale) {
                const uintptr_t q = reinterpret_cast<uintptr_t>(n.g.spk), c = reinterpret_cast<uintptr_t>(n.g.spkCnt);
                const size_t slots = std::max(1u, n.g.numDelaySlots);
                if((a < q + (size_t)r->batch * slots * n.g.numNeurons * sizeof(uint32_t) && q < b) || (a < c + (size_t)r->batch * slots * sizeof(uint32_t) && c < b)) { r->bitmapsStale = true; }
            }
            if(n.g.model != GENNMI_NEURON_SPIKE_SOURCE_ARRAY || r->sourcesStale) { continue; }
            const size_t perNeuron = (size_t)r->batch * n.g.numNeurons * sizeof(uint32_t);
            const uintptr_t st = reinterpret_cast<uintptr_t>(n.g.startSpike), en = reinterpret_cast<uintptr_t>(n.g.endSpike);
            if((a < st + perNeuron && st < b) || (a < en + perNeuron && en < b) || (a < reinterpret_cast<uintptr_t>(n.g.spikeTimes) + n.spikeTimesBytes && reinterpret_cast<uintptr_t>(n.g.spikeTimes) < b)) { r->sourcesStale = true; }
        }
        if(!r->finalised) { continue; }
        for(size_t k = 0; k < r->pre.size(); k++) {
            const auto &p = r->pre[k];
            if(p.g.matrix != GENNMI_MATRIX_SPARSE) { continue; }
            const size_t entries = (size_t)p.g.numSrcNeurons * p.g.rowStride;
            // connectivity (rowLength, ind, d) feeds the segment boundaries of the tile path, the zero-delay lists of the
            // single-launch step, the column views of ordered accumulation and the resident plan's segment tables; weights
            // are copied only into the latter
            const struct { const void *ptr; size_t size; bool connectivity; } arrays[] = {
                {p.g.g, entries * sizeof(float), false}, {p.g.ind, entries * sizeof(uint32_t), true}, {p.g.d, p.g.d ? entries : 0, true},
                {p.g.rowLength, (size_t)p.g.numSrcNeurons * sizeof(uint32_t), true}};
            for(const auto &arr : arrays) {
                const uintptr_t lo = reinterpret_cast<uintptr_t>(arr.ptr);
                if(arr.ptr && arr.size && a < lo + arr.size && lo < b) {
                    if(r->resident) { r->resStale = true; r->resStaleProj.resize(r->pre.size(), 0); r->resStaleProj[k] = 1; }
                    if(arr.connectivity) { r->tablesStale = true; }
                    if(!r->recordTables.empty()) { r->recordsStale = true; }
                }
            }
        }
    }
}

// Step queue.  A caller that advances the model one gennmi_step() at a time (the reference's Runtime::stepTime does) would
// pay a launch per step; a runner on the resident plan can do many steps in one launch.  With a queue enabled, gennmi_step()
// only notes the step; the noted steps run, as one launch where they can, before anything could observe the difference:
// every entry point of the library that reads, writes or frees device memory, synchronises, reads counters or steps by another
// route first executes what is queued (flushQueuedSteps), and so does the queue reaching its limit.
static std::atomic<int> g_queuedRunners{0};
static int flushRunner(gennmi_runner *r);
static int flushPrograms();             // the noted calls of programs (generated kernels), genn_mi355x_program.h
static int checkPrograms();
static int flushQueuedSteps()
{
    { const int rc = flushPrograms(); if(rc) { return rc; } }
    if(g_queuedRunners.load(std::memory_order_relaxed) == 0) { return GENNMI_OK; }
    std::vector<gennmi_runner*> runners;
    {
        std::lock_guard<std::mutex> lock(g_runnersMutex);
        runners = g_runners;
    }
    for(gennmi_runner *r : runners) {
        const int rc = flushRunner(r);
        if(rc) { return rc; }
    }
    return GENNMI_OK;
}
#define FLUSH_QUEUED() do { const int rcFlush_ = flushQueuedSteps(); if(rcFlush_) { return rcFlush_; } } while(0)

namespace gennmi_detail
{
// error reporting and write tracking for the library's other translation units
int fail(int code, const std::string &msg) { return ::fail(code, msg); }
void noteDeviceWrite(const void *dev, size_t bytes) { ::noteDeviceWrite(dev, bytes); }
int flushQueuedSteps() { return ::flushQueuedSteps(); }
int prepareStaticScratch();             // looks up the current device's copy of the static counter array (defined with it)
}

extern "C" {

const char *gennmi_last_error(void) { return g_lastError.c_str(); }

int gennmi_init(int device)
{
    int count = 0;
    HIP_TRY(hipGetDeviceCount(&count));
    if(device < 0 || device >= count) { return fail(GENNMI_EINVAL, "gennmi_init: no such device"); }
    HIP_TRY(hipSetDevice(device));
    hipDeviceProp_t prop;
    HIP_TRY(hipGetDeviceProperties(&prop, device));
    if(prop.warpSize != WAVE) { return fail(GENNMI_EUNSUPPORTED, "gennmi_init: kernels assume 64-wide wavefronts"); }
    return gennmi_detail::prepareStaticScratch();
}

int gennmi_device_name(char *buf, size_t len)
{
    int device = 0;
    HIP_TRY(hipGetDevice(&device));
    hipDeviceProp_t prop;
    HIP_TRY(hipGetDeviceProperties(&prop, device));
    snprintf(buf, len, "%s (%s, %d CUs)", prop.name, prop.gcnArchName, prop.multiProcessorCount);
    return GENNMI_OK;
}

int gennmi_malloc(void **devPtr, size_t bytes)
{
    HIP_TRY(hipMalloc(devPtr, bytes ? bytes : 4));
    return GENNMI_OK;
}
int gennmi_host_malloc(void **hostPtr, size_t bytes, int zeroCopy, void **devPtr)
{
    if(!hostPtr || (zeroCopy && !devPtr)) { return fail(GENNMI_EINVAL, "host_malloc: null result pointer"); }
    HIP_TRY(hipHostMalloc(hostPtr, bytes ? bytes : 4, zeroCopy ? hipHostMallocMapped : hipHostMallocPortable));
    std::memset(*hostPtr, 0, bytes);
    if(devPtr) { *devPtr = nullptr; }
    if(zeroCopy) { HIP_TRY(hipHostGetDevicePointer(devPtr, *hostPtr, 0)); }
    return GENNMI_OK;
}
int gennmi_host_free(void *hostPtr)
{
    if(hostPtr) { HIP_TRY(hipHostFree(hostPtr)); }
    return GENNMI_OK;
}
int gennmi_free(void *devPtr) { FLUSH_QUEUED(); HIP_TRY(hipFree(devPtr)); return GENNMI_OK; }
int gennmi_memcpy_to_device(void *dev, const void *host, size_t bytes)
{
    FLUSH_QUEUED();
    HIP_TRY(hipMemcpy(dev, host, bytes, hipMemcpyHostToDevice));
    noteDeviceWrite(dev, bytes);
    return GENNMI_OK;
}
int gennmi_memcpy_from_device(void *host, const void *dev, size_t bytes)
{
    FLUSH_QUEUED();
    HIP_TRY(hipMemcpy(host, dev, bytes, hipMemcpyDeviceToHost));
    return checkPrograms();         // (the copy waited for every program's stream: their error flags are in host memory)
}
int gennmi_note_device_write(const void *dev, size_t bytes)
{
    FLUSH_QUEUED();
    if(!dev) { return fail(GENNMI_EINVAL, "note_device_write: null pointer"); }
    noteDeviceWrite(dev, bytes);
    return GENNMI_OK;
}
int gennmi_memset(void *dev, int value, size_t bytes)
{
    FLUSH_QUEUED();
    HIP_TRY(hipMemset(dev, value, bytes));
    noteDeviceWrite(dev, bytes);
    return GENNMI_OK;
}
int gennmi_fill_f32(float *dev, float value, size_t count)
{
    FLUSH_QUEUED();
    if(count) {
        fillKernel<<<dim3((unsigned int)((count + BLOCK - 1) / BLOCK)), dim3(BLOCK), 0, 0>>>(dev, value, count);
        HIP_TRY(hipGetLastError());
        HIP_TRY(hipDeviceSynchronize());
        noteDeviceWrite(dev, count * sizeof(float));
    }
    return GENNMI_OK;
}
int gennmi_copy_f32(float *dst, const float *src, size_t count)
{
    FLUSH_QUEUED();
    if(count) {
        if(!dst || !src) { return fail(GENNMI_EINVAL, "copy_f32: null pointer"); }
        const size_t lanes = (count + 3) / 4;
        copyKernel<<<dim3((unsigned int)((lanes + BLOCK - 1) / BLOCK)), dim3(BLOCK), 0, 0>>>(dst, src, count);
        HIP_TRY(hipGetLastError());
        HIP_TRY(hipDeviceSynchronize());
        noteDeviceWrite(dst, count * sizeof(float));
    }
    return GENNMI_OK;
}
int gennmi_synchronize(void) { FLUSH_QUEUED(); HIP_TRY(hipDeviceSynchronize()); return checkPrograms(); }
int gennmi_flush(void) { FLUSH_QUEUED(); return GENNMI_OK; }

// ---- host mirrors: host buffer <-> device buffer pairs, for callers whose generated code only knows host pointers
namespace
{
// deviceInitialised: a device generator filled the buffer since initialisation began, so the host copy is not the one to
// upload; hostStale: ... and has not been copied back since.  releaseHost: the host side is lazily committed address space
// (an array the model places on the device only) whose pages are given back after every upload.
// zeroCopy: host and device side are the same pinned memory (VarLocation::HOST_DEVICE_ZERO_COPY): nothing is ever copied.
struct Mirror { void *dev; size_t bytes; bool deviceInitialised = false, hostStale = false, releaseHost = false, zeroCopy = false; };
std::map<uintptr_t, Mirror> g_mirrors;      // keyed by host base address
std::mutex g_mirrorMutex;
// the registered buffer `host` points into (g_mirrorMutex held)
Mirror *findMirror(const void *host, uintptr_t *base = nullptr)
{
    const uintptr_t h = reinterpret_cast<uintptr_t>(host);
    auto it = g_mirrors.upper_bound(h);
    if(it == g_mirrors.begin()) { return nullptr; }
    --it;
    if(h - it->first >= it->second.bytes) { return nullptr; }
    if(base) { *base = it->first; }
    return &it->second;
}
}
int gennmi_register_mirror(const void *host, void *dev, size_t bytes)
{
    if(!host || !dev || bytes == 0) { return fail(GENNMI_EINVAL, "register_mirror: null pointer or empty buffer"); }
    std::lock_guard<std::mutex> lock(g_mirrorMutex);
    Mirror m{dev, bytes};
    hipPointerAttribute_t attributes{};
    if(hipPointerGetAttributes(&attributes, dev) == hipSuccess) { m.zeroCopy = (attributes.type == hipMemoryTypeHost); }
    else { (void)hipGetLastError(); }
    g_mirrors[reinterpret_cast<uintptr_t>(host)] = m;
    return GENNMI_OK;
}
int gennmi_register_device_array(const void *host, void *dev, size_t bytes)
{
    if(int rc = gennmi_register_mirror(host, dev, bytes)) { return rc; }
    if(reinterpret_cast<uintptr_t>(host) % 4096 != 0) { return fail(GENNMI_EINVAL, "register_device_array: the host range must start on a page boundary"); }
    std::lock_guard<std::mutex> lock(g_mirrorMutex);
    g_mirrors[reinterpret_cast<uintptr_t>(host)].releaseHost = true;
    return GENNMI_OK;
}
int gennmi_mirrors_begin_initialisation(void)
{
    std::lock_guard<std::mutex> lock(g_mirrorMutex);
    for(auto &m : g_mirrors) { m.second.deviceInitialised = m.second.hostStale = false; }
    return GENNMI_OK;
}
int gennmi_mirror_device_initialised(const void *host)
{
    if(!host) { return GENNMI_OK; }
    std::lock_guard<std::mutex> lock(g_mirrorMutex);
    Mirror *m = findMirror(host);
    if(!m) { return fail(GENNMI_EINVAL, "mirror_device_initialised: host pointer is not inside a registered buffer"); }
    m->deviceInitialised = m->hostStale = true;
    return GENNMI_OK;
}
int gennmi_mirror_ensure_host(const void *host)
{
    if(!host) { return GENNMI_OK; }
    FLUSH_QUEUED();
    std::lock_guard<std::mutex> lock(g_mirrorMutex);
    uintptr_t base = 0;
    Mirror *m = findMirror(host, &base);
    if(!m) { return fail(GENNMI_EINVAL, "mirror_ensure_host: host pointer is not inside a registered buffer"); }
    if(m->hostStale && m->zeroCopy) { HIP_TRY(hipDeviceSynchronize()); m->hostStale = false; }
    if(m->hostStale) {
        HIP_TRY(hipMemcpy(reinterpret_cast<void*>(base), m->dev, m->bytes, hipMemcpyDeviceToHost));
        m->hostStale = false;
    }
    return GENNMI_OK;
}
int gennmi_unregister_mirror(const void *host)
{
    std::lock_guard<std::mutex> lock(g_mirrorMutex);
    if(g_mirrors.erase(reinterpret_cast<uintptr_t>(host)) == 0) { return fail(GENNMI_EINVAL, "unregister_mirror: unknown host pointer"); }
    return GENNMI_OK;
}
int gennmi_mirror_device_pointer(const void *host, void **dev)
{
    if(!dev) { return fail(GENNMI_EINVAL, "mirror_device_pointer: null result pointer"); }
    *dev = nullptr;
    if(!host) { return GENNMI_OK; }        // absent arrays stay absent
    std::lock_guard<std::mutex> lock(g_mirrorMutex);
    const uintptr_t h = reinterpret_cast<uintptr_t>(host);
    auto it = g_mirrors.upper_bound(h);
    if(it == g_mirrors.begin()) { return fail(GENNMI_EINVAL, "mirror_device_pointer: host pointer is not inside a registered buffer"); }
    --it;
    if(h - it->first >= it->second.bytes) { return fail(GENNMI_EINVAL, "mirror_device_pointer: host pointer is not inside a registered buffer"); }
    *dev = static_cast<char*>(it->second.dev) + (h - it->first);
    return GENNMI_OK;
}
int gennmi_note_mirror_write(const void *host)
{
    FLUSH_QUEUED();
    if(!host) { return GENNMI_OK; }         // absent arrays stay absent
    Mirror m{nullptr, 0};
    {
        std::lock_guard<std::mutex> lock(g_mirrorMutex);
        const uintptr_t h = reinterpret_cast<uintptr_t>(host);
        auto it = g_mirrors.upper_bound(h);
        if(it == g_mirrors.begin()) { return fail(GENNMI_EINVAL, "note_mirror_write: host pointer is not inside a registered buffer"); }
        --it;
        if(h - it->first >= it->second.bytes) { return fail(GENNMI_EINVAL, "note_mirror_write: host pointer is not inside a registered buffer"); }
        m = it->second;
    }
    noteDeviceWrite(m.dev, m.bytes);
    return GENNMI_OK;
}
int gennmi_push_mirrors(void)
{
    FLUSH_QUEUED();
    std::lock_guard<std::mutex> lock(g_mirrorMutex);
    for(const auto &m : g_mirrors) {
        if(!m.second.deviceInitialised && !m.second.zeroCopy) {
            HIP_TRY(hipMemcpy(m.second.dev, reinterpret_cast<const void*>(m.first), m.second.bytes, hipMemcpyHostToDevice));
            noteDeviceWrite(m.second.dev, m.second.bytes);
        }
        if(m.second.releaseHost) {
            // the pages come back as zeros when next touched; what the model keeps is on the device
            const size_t whole = m.second.bytes / 4096 * 4096;
            if(whole && madvise(reinterpret_cast<void*>(m.first), whole, MADV_DONTNEED) != 0) { return fail(GENNMI_EINVAL, "push_mirrors: madvise failed"); }
        }
    }
    return GENNMI_OK;
}
extern "C++" {
namespace
{
// roctx, if the process can load it (profilers bring it; nothing links against it)
struct Roctx { int (*push)(const char*) = nullptr; int (*pop)() = nullptr; };
const Roctx &roctx()
{
    static const Roctx r = [] {
        Roctx x;
        for(const char *name : {"libroctx64.so.4", "libroctx64.so", "librocprofiler-sdk-roctx.so.1"}) {
            if(void *lib = dlopen(name, RTLD_NOW | RTLD_GLOBAL)) {
                x.push = reinterpret_cast<int(*)(const char*)>(dlsym(lib, "roctxRangePushA"));
                x.pop = reinterpret_cast<int(*)()>(dlsym(lib, "roctxRangePop"));
                if(x.push && x.pop) { break; }
                x = Roctx{};
            }
        }
        return x;
    }();
    return r;
}
}
}   // extern "C++"
int gennmi_profiler_range_push(const char *name)
{
    if(name && roctx().push) { roctx().push(name); }
    return GENNMI_OK;
}
int gennmi_profiler_range_pop(void)
{
    if(roctx().pop) { roctx().pop(); }
    return GENNMI_OK;
}
int gennmi_free_device_memory_bytes(size_t *bytes)
{
    size_t total = 0;
    HIP_TRY(hipMemGetInfo(bytes, &total));
    return GENNMI_OK;
}

int gennmi_abi_struct_sizes(size_t sizes[5])
{
    if(!sizes) { return fail(GENNMI_EINVAL, "abi_struct_sizes: null argument"); }
    sizes[0] = sizeof(gennmi_psm_t); sizes[1] = sizeof(gennmi_cs_t); sizes[2] = sizeof(gennmi_neuron_update_group_t);
    sizes[3] = sizeof(gennmi_presynaptic_update_group_t); sizes[4] = sizeof(gennmi_postsynaptic_update_group_t);
    return GENNMI_OK;
}

int gennmi_runner_create(gennmi_runner **runner, float dt, uint32_t batchSize)
{
    if(!runner || batchSize == 0 || batchSize > 65535) { return fail(GENNMI_EINVAL, "gennmi_runner_create: bad arguments"); }
    gennmi_runner *r = new gennmi_runner;
    r->dt = dt; r->batch = batchSize;
    HIP_TRY(hipStreamCreate(&r->stream));       // blocking stream: ordered against null-stream copies

    // the error flag: one pinned host word, which the kernels reach through its device address (raiseErrorFlag)
    HIP_TRY(hipHostMalloc(reinterpret_cast<void**>(&r->hError), sizeof(uint32_t), hipHostMallocMapped | hipHostMallocCoherent));
    *r->hError = 0;
    HIP_TRY(hipHostGetDevicePointer(reinterpret_cast<void**>(&r->dError), r->hError, 0));
    HIP_TRY(hipMalloc(&r->dEvents, sizeof(unsigned long long) * EVENT_SLOTS * EVENT_SLOT_STRIDE));
    HIP_TRY(hipMemset(r->dEvents, 0, sizeof(unsigned long long) * EVENT_SLOTS * EVENT_SLOT_STRIDE));
    HIP_TRY(hipMalloc(&r->dState, sizeof(StepState)));
    HIP_TRY(hipMemset(r->dState, 0, sizeof(StepState)));
    {
        std::lock_guard<std::mutex> lock(g_runnersMutex);
        g_runners.push_back(r);
    }
    *runner = r;
    return GENNMI_OK;
}

int gennmi_runner_destroy(gennmi_runner *r)
{
    if(!r) { return GENNMI_OK; }
    if(!r->queued.empty()) { r->queued.clear(); g_queuedRunners--; }      // nothing can observe these steps any more
    {
        std::lock_guard<std::mutex> lock(g_runnersMutex);
        g_runners.erase(std::remove(g_runners.begin(), g_runners.end(), r), g_runners.end());
    }
    hipStreamSynchronize(r->stream);
    if(r->graphExec) { hipGraphExecDestroy(r->graphExec); }
    for(hipEvent_t e : r->eventPool) { hipEventDestroy(e); }
    for(hipEvent_t e : r->marks) { if(e) { hipEventDestroy(e); } }
    for(void *q : r->owned) { hipFree(q); }
    for(void *q : r->zeroOwned) { hipFree(q); }
    for(void *q : r->orderedOwned) { hipFree(q); }
    hipFree(r->dOrderedSources); hipFree(r->dOrderedBitmaps);
    hipFree(r->dTile); hipFree(r->dConvTile);
    hipFree(r->dNeuron); hipFree(r->dPre); hipFree(r->dPost); hipFree(r->dDense); hipFree(r->dProc); hipFree(r->dAgg); if(r->hError) { hipHostFree(r->hError); } hipFree(r->dEvents); hipFree(r->dState);
    hipStreamDestroy(r->stream);
    delete r;
    return GENNMI_OK;
}

int gennmi_push_neuron_update_group(gennmi_runner *r, const gennmi_neuron_update_group_t *g, uint32_t *idx)
{
    if(!r || !g) { return fail(GENNMI_EINVAL, "push_neuron_update_group: null argument"); }
    if(r->finalised) { return fail(GENNMI_ESTATE, "push_neuron_update_group: runner already finalised"); }
    if(g->numNeurons == 0) { return fail(GENNMI_EINVAL, "push_neuron_update_group: empty population"); }
    if(g->numPSM > GENNMI_MAX_PSM || g->numCS > GENNMI_MAX_CS) { return fail(GENNMI_EUNSUPPORTED, "push_neuron_update_group: too many children"); }
    if(!g->spk || !g->spkCnt) { return fail(GENNMI_EINVAL, "push_neuron_update_group: spike queue missing"); }
    if(g->numDelaySlots > 1 && (g->numExtraSpk || g->preTrace || g->postTrace || g->sT)) {
        return fail(GENNMI_EUNSUPPORTED, "push_neuron_update_group: axonal delay slots together with plasticity or further spike arrays");
    }
    if(g->model == GENNMI_NEURON_SPIKE_SOURCE_ARRAY) {
        if(!g->startSpike || !g->endSpike || !g->spikeTimes) { return fail(GENNMI_EINVAL, "push_neuron_update_group: spike source arrays missing"); }
    }
    else if(g->model == GENNMI_NEURON_LIF || g->model == GENNMI_NEURON_IZHIKEVICH) {
        if(!g->var0 || !g->var1) { return fail(GENNMI_EINVAL, "push_neuron_update_group: state variables missing"); }
    }
    else { return fail(GENNMI_EUNSUPPORTED, "push_neuron_update_group: unknown neuron model"); }
    for(uint32_t m = 0; m < g->numPSM; m++) {
        if(!g->psm[m].outPost) { return fail(GENNMI_EINVAL, "push_neuron_update_group: outPost missing"); }
        if(g->psm[m].maxDenDelay && !g->psm[m].denDelay) { return fail(GENNMI_EINVAL, "push_neuron_update_group: denDelay missing"); }
        if(g->psm[m].kind > GENNMI_PSM_DELTACURR) { return fail(GENNMI_EUNSUPPORTED, "push_neuron_update_group: unknown postsynaptic model"); }
    }
    for(uint32_t c = 0; c < g->numCS; c++) {
        if(g->cs[c].kind == GENNMI_CS_ARRAY && (!g->cs[c].array || g->cs[c].arraySteps == 0)) { return fail(GENNMI_EINVAL, "push_neuron_update_group: current-source array missing"); }
        if(g->cs[c].kind == GENNMI_CS_POISSON_EXP && !g->cs[c].current) { return fail(GENNMI_EINVAL, "push_neuron_update_group: PoissonExp state missing"); }
        if(g->cs[c].kind > GENNMI_CS_POISSON_EXP) { return fail(GENNMI_EUNSUPPORTED, "push_neuron_update_group: unknown current source"); }
    }
    if(g->numExtraSpk > GENNMI_MAX_EXTRA_SPK) { return fail(GENNMI_EUNSUPPORTED, "push_neuron_update_group: too many spike arrays"); }
    for(uint32_t q = 0; q < g->numExtraSpk; q++) {
        if(!g->extraSpkCnt[q] || !g->extraSpk[q]) { return fail(GENNMI_EINVAL, "push_neuron_update_group: extra spike array missing"); }
    }
    if(g->numPreOutput > GENNMI_MAX_PRE_OUTPUT) { return fail(GENNMI_EUNSUPPORTED, "push_neuron_update_group: too many presynaptic outputs"); }
    if(g->numPreOutput && g->model == GENNMI_NEURON_SPIKE_SOURCE_ARRAY) { return fail(GENNMI_EUNSUPPORTED, "push_neuron_update_group: presynaptic output into a spike source"); }
    for(uint32_t q = 0; q < g->numPreOutput; q++) { if(!g->outPre[q]) { return fail(GENNMI_EINVAL, "push_neuron_update_group: outPre missing"); } }
    if(g->numSpkEvent > GENNMI_MAX_SPK_EVENT) { return fail(GENNMI_EUNSUPPORTED, "push_neuron_update_group: too many spike-like event conditions"); }
    if(g->numSpkEvent && (g->model == GENNMI_NEURON_SPIKE_SOURCE_ARRAY || g->numDelaySlots > 1)) {
        return fail(GENNMI_EUNSUPPORTED, "push_neuron_update_group: spike-like events need a LIF or Izhikevich group without delay slots");
    }
    for(uint32_t e = 0; e < g->numSpkEvent; e++) {
        if(!g->spkEvent[e].spkCntEvent || !g->spkEvent[e].spkEvent) { return fail(GENNMI_EINVAL, "push_neuron_update_group: event queue missing"); }
    }
    NeuronGroupDev d;
    memset(&d, 0, sizeof(d));
    d.g = *g;
    if(idx) { *idx = (uint32_t)r->neuron.size(); }
    r->neuron.push_back(d);
    return GENNMI_OK;
}

int gennmi_push_presynaptic_update_group(gennmi_runner *r, const gennmi_presynaptic_update_group_t *g, uint32_t *idx)
{
    if(!r || !g) { return fail(GENNMI_EINVAL, "push_presynaptic_update_group: null argument"); }
    if(r->finalised) { return fail(GENNMI_ESTATE, "push_presynaptic_update_group: runner already finalised"); }
    if(!g->srcSpk || !g->srcSpkCnt || (!g->outPost && g->wum != GENNMI_WUM_STATIC_PULSE_REVERSE)) { return fail(GENNMI_EINVAL, "push_presynaptic_update_group: required array missing"); }
    if(g->numSrcNeurons == 0 || g->numTrgNeurons == 0) { return fail(GENNMI_EINVAL, "push_presynaptic_update_group: empty population"); }
    if(g->matrix == GENNMI_MATRIX_PROCEDURAL) {
        const gennmi_procedural_t &q = g->procedural;
        if(g->wum != GENNMI_WUM_STATIC_PULSE && g->wum != GENNMI_WUM_STATIC_PULSE_CONSTANT_WEIGHT) {
            return fail(GENNMI_EUNSUPPORTED, "push_presynaptic_update_group: PROCEDURAL supports StaticPulse and StaticPulseConstantWeight");
        }
        if(g->numSrcDelaySlots > 1 || g->axonalDelaySteps) { return fail(GENNMI_EUNSUPPORTED, "push_presynaptic_update_group: axonal delay on a PROCEDURAL projection"); }
        if(g->rowStride == 0 || g->numTrgNeurons > 0x7fffffffu) { return fail(GENNMI_EINVAL, "push_presynaptic_update_group: procedural row stride or target count out of range"); }
        if(q.connectivity > GENNMI_CONNECT_FIXED_NUMBER_POST) { return fail(GENNMI_EUNSUPPORTED, "push_presynaptic_update_group: unknown procedural connectivity"); }
        if(q.connectivity != GENNMI_CONNECT_FIXED_NUMBER_POST && !(q.prob >= 0.0 && q.prob <= 1.0)) { return fail(GENNMI_EINVAL, "push_presynaptic_update_group: connection probability outside [0, 1]"); }
        if(q.connectivity == GENNMI_CONNECT_FIXED_NUMBER_POST && q.num > g->rowStride) { return fail(GENNMI_EINVAL, "push_presynaptic_update_group: num exceeds rowStride"); }
        if(q.weightSnippet > GENNMI_INIT_EXPONENTIAL) { return fail(GENNMI_EUNSUPPORTED, "push_presynaptic_update_group: procedural weights support Constant, Uniform, Normal, NormalClipped and Exponential"); }
        ProcGroupDev pd;
        memset(&pd, 0, sizeof(pd));
        pd.g = *g;
        pd.g.maxDenDelay = 0;
        pd.connectivity = gennmi_rows::Stream{(uint32_t)q.seed, (uint32_t)(q.seed >> 32), q.connectivityStream};
        pd.weight = gennmi_rows::Stream{(uint32_t)q.seed, (uint32_t)(q.seed >> 32), q.weightStream};
        pd.weightInit.snippet = (g->wum == GENNMI_WUM_STATIC_PULSE_CONSTANT_WEIGHT) ? (uint32_t)GENNMI_INIT_CONSTANT : q.weightSnippet;
        for(int k = 0; k < 4; k++) { pd.weightInit.p[k] = (float)q.weightParams[k]; }
        if(g->wum == GENNMI_WUM_STATIC_PULSE_CONSTANT_WEIGHT) { pd.weightInit.p[0] = g->constantWeight; }
        pd.probLogRecip = (q.prob == 0.0) ? -INFINITY : (float)(1.0 / std::log(1.0 - q.prob));
        if(idx) { *idx = (uint32_t)(r->pre.size() + r->dense.size() + r->proc.size()); }
        r->proc.push_back(pd);
        return GENNMI_OK;
    }
    if(g->matrix == GENNMI_MATRIX_DENSE || g->matrix == GENNMI_MATRIX_BITMASK) {
        const bool constant = (g->wum == GENNMI_WUM_STATIC_PULSE_CONSTANT_WEIGHT);
        if(g->matrix == GENNMI_MATRIX_DENSE) {
            if(!constant && g->wum != GENNMI_WUM_STATIC_PULSE) { return fail(GENNMI_EUNSUPPORTED, "push_presynaptic_update_group: DENSE supports StaticPulse and StaticPulseConstantWeight"); }
            if(!constant && !g->g) { return fail(GENNMI_EINVAL, "push_presynaptic_update_group: dense weights missing"); }
        }
        else {
            if(!constant) { return fail(GENNMI_EUNSUPPORTED, "push_presynaptic_update_group: BITMASK needs StaticPulseConstantWeight"); }
            if(!g->gp || g->rowStride < g->numTrgNeurons || (g->rowStride % 32) != 0) {
                return fail(GENNMI_EINVAL, "push_presynaptic_update_group: bitmask words missing or row stride not numTrg padded to 32");
            }
        }
        if(g->numSrcDelaySlots > 1 || g->axonalDelaySteps) { return fail(GENNMI_EUNSUPPORTED, "push_presynaptic_update_group: axonal delay on a DENSE or BITMASK projection"); }
        DenseGroupDev dd;
        memset(&dd, 0, sizeof(dd));
        dd.g = *g;
        dd.g.maxDenDelay = 0;
        if(idx) { *idx = (uint32_t)(r->pre.size() + r->dense.size()); }
        r->dense.push_back(dd);
        return GENNMI_OK;
    }
    if(!g->g) { return fail(GENNMI_EINVAL, "push_presynaptic_update_group: required array missing"); }
    if(g->numSrcDelaySlots > 1) {
        if(g->axonalDelaySteps >= g->numSrcDelaySlots) { return fail(GENNMI_EINVAL, "push_presynaptic_update_group: axonal delay does not fit the source's delay slots"); }
        if(g->wum == GENNMI_WUM_STDP_TRACE || g->wum == GENNMI_WUM_STDP) { return fail(GENNMI_EUNSUPPORTED, "push_presynaptic_update_group: axonal delay on a plastic projection"); }
    }
    else if(g->axonalDelaySteps) { return fail(GENNMI_EINVAL, "push_presynaptic_update_group: axonal delay without delay slots"); }
    PreGroupDev d;
    memset(&d, 0, sizeof(d));
    d.g = *g;
    if(g->matrix == GENNMI_MATRIX_SPARSE) {
        if(!g->rowLength || !g->ind || g->rowStride == 0) { return fail(GENNMI_EINVAL, "push_presynaptic_update_group: sparse arrays missing"); }
        // Synapse ids beyond 32 bits (backendBase.cc:503-522 switches the index type at numPre * rowStride > 2^32 - 1): the scatter
        // and tile paths of a static projection index rows in 64 bits throughout; the views other rules need (column remap,
        // zero-delay lists, segment tables of the resident plan) hold 32-bit ids
        if((uint64_t)g->numSrcNeurons * g->rowStride > 0xFFFFFFFFull && g->wum != GENNMI_WUM_STATIC_PULSE) {
            return fail(GENNMI_EUNSUPPORTED, "push_presynaptic_update_group: synapse index exceeds 32 bits (supported for static projections without delay only)");
        }
        if(g->wum == GENNMI_WUM_STATIC_PULSE_DENDRITIC_DELAY) {
            if(!g->d || !g->denDelay || g->maxDenDelay == 0) { return fail(GENNMI_EINVAL, "push_presynaptic_update_group: dendritic delay arrays missing"); }
        }
        else if(g->wum == GENNMI_WUM_STDP_TRACE) {
            if(!g->trgST || !g->postTrace) { return fail(GENNMI_EINVAL, "push_presynaptic_update_group: STDP arrays missing"); }
        }
        else if(g->wum == GENNMI_WUM_STDP) {
            if(!g->trgST || !(g->tauMinus > 0.0f)) { return fail(GENNMI_EINVAL, "push_presynaptic_update_group: STDP needs the target's spike times and tauMinus > 0"); }
        }
        else if(g->wum == GENNMI_WUM_STATIC_PULSE_REVERSE) {
            if(!g->outPre) { return fail(GENNMI_EINVAL, "push_presynaptic_update_group: outPre missing"); }
        }
        else if(g->wum == GENNMI_WUM_STATIC_GRADED) {
            if(!g->srcV || !(g->gradedVslope != 0.0f)) { return fail(GENNMI_EINVAL, "push_presynaptic_update_group: graded synapses need the source's V and a non-zero Vslope"); }
            if(g->numSrcDelaySlots > 1) { return fail(GENNMI_EUNSUPPORTED, "push_presynaptic_update_group: axonal delay on a graded projection"); }
        }
        else if(g->wum != GENNMI_WUM_STATIC_PULSE) { return fail(GENNMI_EUNSUPPORTED, "push_presynaptic_update_group: unknown weight update model"); }
        if(g->wum != GENNMI_WUM_STATIC_PULSE_DENDRITIC_DELAY) { d.g.maxDenDelay = 0; }
    }
    else if(g->matrix == GENNMI_MATRIX_TOEPLITZ_CONV2D) {
        const int32_t *c = g->conv;
        for(int k = 0; k < 8; k++) { if(c[k] <= 0) { return fail(GENNMI_EINVAL, "push_presynaptic_update_group: bad conv parameter"); } }
        if((uint64_t)c[2] * c[3] * c[4] != g->numSrcNeurons || (uint64_t)c[5] * c[6] * c[7] != g->numTrgNeurons) {
            return fail(GENNMI_EINVAL, "push_presynaptic_update_group: conv shape does not match population sizes");
        }
        if(g->wum != GENNMI_WUM_STATIC_PULSE) { return fail(GENNMI_EUNSUPPORTED, "push_presynaptic_update_group: Toeplitz supports StaticPulse only"); }
        // derived parameters conv_bw / conv_bh (initToeplitzConnectivitySnippet.h:113-114)
        d.convBW = ((c[3] + c[1] - 1) - c[6]) / 2;
        d.convBH = ((c[2] + c[0] - 1) - c[5]) / 2;
        d.g.maxDenDelay = 0;
    }
    else { return fail(GENNMI_EUNSUPPORTED, "push_presynaptic_update_group: unknown matrix type"); }
    if(idx) { *idx = (uint32_t)r->pre.size(); }
    r->pre.push_back(d);
    return GENNMI_OK;
}

int gennmi_push_postsynaptic_update_group(gennmi_runner *r, const gennmi_postsynaptic_update_group_t *g, uint32_t *idx)
{
    if(!r || !g) { return fail(GENNMI_EINVAL, "push_postsynaptic_update_group: null argument"); }
    if(r->finalised) { return fail(GENNMI_ESTATE, "push_postsynaptic_update_group: runner already finalised"); }
    if(!(g->tauPlus >= 0.0f)) { return fail(GENNMI_EINVAL, "push_postsynaptic_update_group: tauPlus must be 0 (trace rule) or positive"); }
    if(!g->colLength || !g->remap || !g->g || !g->trgSpk || !g->trgSpkCnt || !g->srcST || (!g->preTrace && !(g->tauPlus > 0.0f))) {
        return fail(GENNMI_EINVAL, "push_postsynaptic_update_group: required array missing");
    }
    if(g->rowStride == 0 || g->colStride == 0) { return fail(GENNMI_EINVAL, "push_postsynaptic_update_group: zero stride"); }
    if((g->rowLength == nullptr) != (g->ind == nullptr)) { return fail(GENNMI_EINVAL, "push_postsynaptic_update_group: rowLength and ind go together"); }
    PostGroupDev d;
    memset(&d, 0, sizeof(d));
    d.g = *g;
    if(idx) { *idx = (uint32_t)r->post.size(); }
    r->post.push_back(d);
    return GENNMI_OK;
}

// Resident plan (residentKernel): chosen when the whole network fits the chip — batch 1, static SPARSE projections
// (with or without dendritic delay) with ascending rows between LIF / Izhikevich populations driven by DC or PoissonExp sources, every
// tile of 256 neurons with its ring slices in LDS and all tiles resident at once.  GENNMI_RESIDENT=0 disables it.
static int setupResident(gennmi_runner *r, uint32_t numCU)
{
    const char *env = getenv("GENNMI_RESIDENT");
    if(env && atoi(env) == 0) { return GENNMI_OK; }
    if(r->batch != 1 || !r->post.empty() || r->pre.empty() || !r->dense.empty() || !r->proc.empty() || r->neuron.size() > RES_MAX_GROUPS) { return GENNMI_OK; }
    for(const auto &n : r->neuron) {
        const auto &g = n.g;
        if((g.model != GENNMI_NEURON_LIF && g.model != GENNMI_NEURON_IZHIKEVICH) || g.preTrace || g.postTrace || g.sT || g.numDelaySlots > 1 || g.numSpkEvent || g.numPreOutput) { return GENNMI_OK; }
        for(uint32_t c = 0; c < g.numCS; c++) { if(g.cs[c].kind == GENNMI_CS_ARRAY) { return GENNMI_OK; } }
    }
    // tiles and their LDS layout
    std::vector<ResTile> tiles;
    std::vector<uint8_t> tileGroup;
    std::vector<uint32_t> firstTile(r->neuron.size()), numTilesOf(r->neuron.size());
    size_t ldsFloatsMax = 0;
    for(size_t gi = 0; gi < r->neuron.size(); gi++) {
        const auto &g = r->neuron[gi].g;
        ResTile t{};
        uint32_t offset = 0;
        for(uint32_t m = 0; m < g.numPSM; m++) {
            t.ldsIn[m] = offset; offset += RES_T;
            if(g.psm[m].maxDenDelay) { t.ldsRing[m] = offset; offset += g.psm[m].maxDenDelay * RES_T; }
        }
        t.ldsFloats = offset;
        ldsFloatsMax = std::max<size_t>(ldsFloatsMax, offset);
        t.group = (uint32_t)gi;
        t.tilesInGroup = (g.numNeurons + RES_T - 1) / RES_T;
        t.firstTileOfGroup = (uint32_t)tiles.size();
        firstTile[gi] = t.firstTileOfGroup; numTilesOf[gi] = t.tilesInGroup;
        for(uint32_t k = 0; k < t.tilesInGroup; k++) {
            t.tileInGroup = k; t.first = k * RES_T; t.count = std::min<uint32_t>(RES_T, g.numNeurons - t.first);
            tiles.push_back(t);
            tileGroup.push_back((uint8_t)gi);
        }
    }
    if(tiles.empty() || tiles.size() > RES_MAX_TILES) { return GENNMI_OK; }
    const size_t ldsBytes = std::max<size_t>(ldsFloatsMax, 1) * sizeof(float);
    if(ldsBytes > 96 * 1024) { return GENNMI_OK; }
    bool poisson = false;
    for(const auto &n : r->neuron) {
        for(uint32_t c = 0; c < n.g.numCS; c++) { poisson = poisson || n.g.cs[c].kind == GENNMI_CS_POISSON_EXP; }
    }
    const void *kernel = poisson ? reinterpret_cast<const void*>(residentKernel<true>) : reinterpret_cast<const void*>(residentKernel<false>);
    if(ldsBytes > 32 * 1024) {
        HIP_TRY(hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)ldsBytes));
    }
    int perCU = 0;
    if(poisson) { HIP_TRY(hipOccupancyMaxActiveBlocksPerMultiprocessor(&perCU, residentKernel<true>, BLOCK, ldsBytes)); }
    else { HIP_TRY(hipOccupancyMaxActiveBlocksPerMultiprocessor(&perCU, residentKernel<false>, BLOCK, ldsBytes)); }
    if((size_t)perCU * numCU < tiles.size()) { return GENNMI_OK; }

    // projections: source group, target group and postsynaptic model, segment table
    struct Link { size_t src, trg; uint32_t psm; };
    std::vector<Link> links;
    for(const auto &p : r->pre) {
        const auto &q = p.g;
        if(q.matrix != GENNMI_MATRIX_SPARSE || (q.wum != GENNMI_WUM_STATIC_PULSE && q.wum != GENNMI_WUM_STATIC_PULSE_DENDRITIC_DELAY)) { return GENNMI_OK; }
        if((unsigned long long)q.numSrcNeurons * q.rowStride > 0xFFFFFFFFull) { return GENNMI_OK; }
        const bool delayed = (q.wum == GENNMI_WUM_STATIC_PULSE_DENDRITIC_DELAY);
        Link l{r->neuron.size(), r->neuron.size(), 0};
        for(size_t gi = 0; gi < r->neuron.size(); gi++) {
            const auto &g = r->neuron[gi].g;
            if(g.spk == q.srcSpk && g.numNeurons == q.numSrcNeurons) { l.src = gi; }
            if(g.numNeurons != q.numTrgNeurons) { continue; }
            for(uint32_t m = 0; m < g.numPSM; m++) {
                const bool match = delayed ? (g.psm[m].denDelay == q.denDelay && g.psm[m].maxDenDelay == q.maxDenDelay && q.maxDenDelay > 0)
                                           : (g.psm[m].outPost == q.outPost && g.psm[m].maxDenDelay == 0);
                if(match) { l.trg = gi; l.psm = m; }
            }
        }
        if(l.src == r->neuron.size() || l.trg == r->neuron.size()) { return GENNMI_OK; }
        links.push_back(l);
    }
    for(size_t gi = 0; gi < r->neuron.size(); gi++) {
        size_t incoming = 0;
        for(const auto &l : links) { incoming += (l.trg == gi) ? 1 : 0; }
        if(incoming > RES_MAX_PROJ) { return GENNMI_OK; }
    }
    uint32_t *dFlag = nullptr;
    HIP_TRY(hipMalloc(&dFlag, sizeof(uint32_t)));
    HIP_TRY(hipMemset(dFlag, 0, sizeof(uint32_t)));
    for(const auto &p : r->pre) {
        const size_t entries = (size_t)p.g.numSrcNeurons * p.g.rowStride;
        residentSortedKernel<<<dim3((unsigned int)((entries + BLOCK - 1) / BLOCK)), dim3(BLOCK), 0, 0>>>(p.g.numSrcNeurons, p.g.rowStride, p.g.rowLength, p.g.ind, dFlag);
    }
    HIP_TRY(hipGetLastError());
    uint32_t unsorted = 0;
    HIP_TRY(hipMemcpy(&unsorted, dFlag, sizeof(uint32_t), hipMemcpyDeviceToHost));
    HIP_TRY(hipFree(dFlag));
    if(unsorted) { return GENNMI_OK; }
    for(size_t k = 0; k < r->pre.size(); k++) {
        const auto &q = r->pre[k].g;
        const Link &l = links[k];
        const uint32_t tilesInGroup = numTilesOf[l.trg];
        const size_t entries = (size_t)q.numSrcNeurons * tilesInGroup;
        if(q.rowStride > 0xFFFFu) { return GENNMI_OK; }         // a segment's length is a 16-bit field (device allocations made so far stay owned)
        u32x4 *dSeg = nullptr;
        HIP_TRY(hipMalloc(&dSeg, entries * 2 * sizeof(u32x4)));
        r->owned.push_back(dSeg);
        const uint32_t depth = (q.wum == GENNMI_WUM_STATIC_PULSE_DENDRITIC_DELAY) ? q.maxDenDelay : 0u;
        residentSegKernel<<<dim3((unsigned int)((entries + BLOCK - 1) / BLOCK)), dim3(BLOCK), 0, 0>>>(q.numSrcNeurons, q.rowStride, q.rowLength, q.ind, q.g, q.d,
                                                                                                     depth, tilesInGroup, dSeg);
        r->resSegs.push_back(dSeg);
        r->resSegTiles.push_back(tilesInGroup);
        HIP_TRY(hipGetLastError());
        const size_t padded = (size_t)q.numSrcNeurons * q.rowStride;
        u32x2 *dPacked = nullptr;
        if(hipMalloc(&dPacked, std::max<size_t>(padded, 1) * sizeof(u32x2)) != hipSuccess) {
            (void)hipGetLastError();            // no room for the second copy of the synapses: the network steps with the other plans
            return GENNMI_OK;
        }
        r->owned.push_back(dPacked);
        if(padded) {
            residentPackKernel<<<dim3((unsigned int)((padded + BLOCK - 1) / BLOCK)), dim3(BLOCK), 0, 0>>>(padded, q.ind, q.g, depth ? q.d : nullptr, dPacked);
            HIP_TRY(hipGetLastError());
        }
        r->resPacked.push_back(dPacked);
        ResProj proj{};
        proj.packed = dPacked; proj.seg = dSeg;
        proj.D = (q.wum == GENNMI_WUM_STATIC_PULSE_DENDRITIC_DELAY) ? q.maxDenDelay : 0u;
        proj.magic = proj.D ? (uint32_t)(0x100000000ull / proj.D) + 1u : 0u;
        proj.srcGroup = (uint32_t)l.src;
        for(uint32_t t = firstTile[l.trg]; t < firstTile[l.trg] + tilesInGroup; t++) {
            proj.lds = proj.D ? tiles[t].ldsRing[l.psm] : tiles[t].ldsIn[l.psm];
            tiles[t].proj[tiles[t].numProj++] = proj;
        }
    }
    auto upload = [r](void **dst, const void *src, size_t bytes) -> hipError_t {
        hipError_t e = hipMalloc(dst, bytes);
        if(e != hipSuccess) { return e; }
        r->owned.push_back(*dst);
        return hipMemcpy(*dst, src, bytes, hipMemcpyHostToDevice);
    };
    std::vector<NeuronGroupDev> groups(r->neuron.begin(), r->neuron.end());
    HIP_TRY(upload((void**)&r->dResTiles, tiles.data(), tiles.size() * sizeof(ResTile)));
    HIP_TRY(upload((void**)&r->dResGroups, groups.data(), groups.size() * sizeof(NeuronGroupDev)));
    HIP_TRY(upload((void**)&r->dResTileGroup, tileGroup.data(), tileGroup.size()));
    r->resReplicaStride = (uint32_t)((2 * tiles.size() + 511) / 512 * 512);          // in words: copies start 4 KiB-aligned
    HIP_TRY(hipMalloc(&r->dResTags, (size_t)RES_REPLICAS * r->resReplicaStride * sizeof(unsigned long long)));
    r->owned.push_back(r->dResTags);
    // cleared once: sequence number 0 is the one no work-group ever waits for before it has come round again
    HIP_TRY(hipMemset(r->dResTags, 0, (size_t)RES_REPLICAS * r->resReplicaStride * sizeof(unsigned long long)));
    r->resSeq = 0;
    HIP_TRY(hipMalloc(&r->dResSide, 2 * tiles.size() * RES_T * sizeof(unsigned long long)));
    r->owned.push_back(r->dResSide);
    // (cleared once as well: its entries name their exchange by the unwrapped sequence number, which starts at 1)
    HIP_TRY(hipMemset(r->dResSide, 0, 2 * tiles.size() * RES_T * sizeof(unsigned long long)));
    r->resTiles = (uint32_t)tiles.size();
    r->resLdsBytes = ldsBytes;
    r->resPoisson = poisson;
    r->resident = true;
    return GENNMI_OK;
}

// `numSteps` steps of a network on the resident plan, as few launches as the sequence counter allows
static int launchResident(gennmi_runner *r, unsigned long long timestep, unsigned long long numSteps, unsigned long long numRecordingTimesteps)
{
    constexpr unsigned long long MAX_STEPS = 1ull << 20;
    if(*r->hError) { return fail(GENNMI_EDEVICE, "a kernel's bounded wait for other work-groups expired earlier; the runner's state is undefined"); }
    bool stale;
    std::vector<uint8_t> staleProj;
    {
        std::lock_guard<std::mutex> lock(g_runnersMutex);
        stale = r->resStale;
        r->resStale = false;
        staleProj.swap(r->resStaleProj);
    }
    if(stale) {
        // weights or connectivity of these projections were written since their segment tables and packed records were built
        for(size_t k = 0; k < r->pre.size(); k++) {
            if(k >= staleProj.size() || !staleProj[k]) { continue; }
            const auto &q = r->pre[k].g;
            const size_t entries = (size_t)q.numSrcNeurons * r->resSegTiles[k];
            const uint32_t depth = (q.wum == GENNMI_WUM_STATIC_PULSE_DENDRITIC_DELAY) ? q.maxDenDelay : 0u;
            residentSegKernel<<<dim3((unsigned int)((entries + BLOCK - 1) / BLOCK)), dim3(BLOCK), 0, r->stream>>>(
                q.numSrcNeurons, q.rowStride, q.rowLength, q.ind, q.g, q.d, depth, r->resSegTiles[k], r->resSegs[k]);
            const size_t padded = (size_t)q.numSrcNeurons * q.rowStride;
            if(padded) {
                residentPackKernel<<<dim3((unsigned int)((padded + BLOCK - 1) / BLOCK)), dim3(BLOCK), 0, r->stream>>>(padded, q.ind, q.g, depth ? q.d : nullptr, r->resPacked[k]);
            }
        }
        HIP_TRY(hipGetLastError());
    }
    for(unsigned long long done = 0; done < numSteps; ) {
        const uint32_t chunk = (uint32_t)std::min(MAX_STEPS, numSteps - done);
        auto launch = r->resPoisson ? residentKernel<true> : residentKernel<false>;
        launch<<<dim3(r->resTiles), dim3(BLOCK), r->resLdsBytes, r->stream>>>(
            r->dResTiles, r->resTiles, r->dResGroups, r->dResTileGroup, r->dResTags, r->dResSide, timestep + done, r->epoch, numRecordingTimesteps,
            chunk, r->dt, r->fusedStep ? 1u : 0u, r->dError, r->dEvents, r->resReplicaStride, r->resSeq);
        HIP_TRY(hipGetLastError());
        r->resSeq += chunk + 1u;                                   // the launch used sequence numbers resSeq + 1 ... resSeq + chunk + 1 (words hold them modulo 2^23)
        done += chunk;
        r->epoch += chunk;
    }
    return GENNMI_OK;
}

// Single-launch step: shadow spike queues and, per population, the list of outgoing synapses whose delay is a multiple of
// the ring depth (delivered by the neuron update of the spiking neuron).  Called at finalise and again whenever the
// connectivity has been rewritten; the caller then uploads the descriptor tables.
static int buildZeroDelayLists(gennmi_runner *r)
{
    for(void *q : r->zeroOwned) { hipFree(q); }
    r->zeroOwned.clear();
    auto devAlloc = [](std::vector<void*> &owner, void **q, size_t bytes) -> hipError_t {
        hipError_t e = hipMalloc(q, bytes ? bytes : 4);
        if(e == hipSuccess) { owner.push_back(*q); e = hipMemset(*q, 0, bytes ? bytes : 4); }
        return e;
    };
    for(auto &n : r->neuron) {
        if(!n.shadowSpk) {
            HIP_TRY(devAlloc(r->owned, (void**)&n.shadowSpk, 2 * (size_t)r->batch * n.g.numNeurons * sizeof(uint32_t)));
            HIP_TRY(devAlloc(r->owned, (void**)&n.shadowCnt, 2 * (size_t)r->batch * sizeof(uint32_t)));
        }
        std::vector<PreGroupDev*> outs;
        for(auto &p : r->pre) { if(p.g.srcSpk == n.g.spk) { outs.push_back(&p); } }
        if(outs.empty()) { continue; }
        const uint32_t N = n.g.numNeurons;
        const dim3 grid((N + BLOCK - 1) / BLOCK);
        uint32_t *dLen = nullptr;
        HIP_TRY(devAlloc(r->zeroOwned, (void**)&dLen, (size_t)N * sizeof(uint32_t)));
        std::vector<std::vector<uint32_t>> len(outs.size(), std::vector<uint32_t>(N));
        for(size_t o = 0; o < outs.size(); o++) {
            const auto &q = outs[o]->g;
            zeroDelayScanKernel<<<grid, dim3(BLOCK), 0, 0>>>(N, q.rowStride, q.rowLength, q.d, q.maxDenDelay, q.ind, q.g, q.denDelay,
                                                             q.numTrgNeurons, dLen, nullptr, nullptr);
            HIP_TRY(hipGetLastError());
            HIP_TRY(hipMemcpy(len[o].data(), dLen, (size_t)N * sizeof(uint32_t), hipMemcpyDeviceToHost));
        }
        std::vector<uint32_t> start(N + 1, 0);
        for(uint32_t i = 0; i < N; i++) {
            uint64_t sum = start[i];
            for(size_t o = 0; o < outs.size(); o++) { sum += len[o][i]; }
            if(sum > 0xFFFFFFFFull) { return fail(GENNMI_EUNSUPPORTED, "runner_finalise: too many zero-delay synapses"); }
            start[i + 1] = (uint32_t)sum;
        }
        uint32_t *dStart = nullptr, *dOffset = nullptr; ZeroDelayEntry *dEntries = nullptr;
        HIP_TRY(devAlloc(r->zeroOwned, (void**)&dStart, (size_t)(N + 1) * sizeof(uint32_t)));
        HIP_TRY(hipMemcpy(dStart, start.data(), (size_t)(N + 1) * sizeof(uint32_t), hipMemcpyHostToDevice));
        HIP_TRY(devAlloc(r->zeroOwned, (void**)&dOffset, (size_t)N * sizeof(uint32_t)));
        HIP_TRY(devAlloc(r->zeroOwned, (void**)&dEntries, (size_t)std::max(1u, start[N]) * sizeof(ZeroDelayEntry)));
        std::vector<uint32_t> offset(start.begin(), start.begin() + N);
        for(size_t o = 0; o < outs.size(); o++) {
            auto &q = outs[o]->g;
            HIP_TRY(hipMemcpy(dOffset, offset.data(), (size_t)N * sizeof(uint32_t), hipMemcpyHostToDevice));
            zeroDelayScanKernel<<<grid, dim3(BLOCK), 0, 0>>>(N, q.rowStride, q.rowLength, q.d, q.maxDenDelay, q.ind, q.g, q.denDelay,
                                                             q.numTrgNeurons, nullptr, dOffset, dEntries);
            HIP_TRY(hipGetLastError());
            HIP_TRY(hipDeviceSynchronize());
            for(uint32_t i = 0; i < N; i++) { offset[i] += len[o][i]; }
            outs[o]->skipZeroDelay = 1; outs[o]->shadowSpk = n.shadowSpk; outs[o]->shadowCnt = n.shadowCnt;
        }
        n.zeroStart = dStart; n.zeroEntries = dEntries;
    }
    return GENNMI_OK;
}

// Single-launch step: where the zero-delay synapses of the last completed step's spikes have been delivered, keyed by
// (weight address, batch) — one entry per synapse and batch
static int pendingZeroDelay(gennmi_runner *r, std::map<std::pair<const float*, uint32_t>, float*> &out)
{
    if(r->epoch == 0) { return GENNMI_OK; }
    const uint32_t parity = (uint32_t)((r->epoch + 1) & 1);         // the queue the coming step's presynaptic update reads
    for(const auto &n : r->neuron) {
        if(!n.zeroStart) { continue; }
        const uint32_t N = n.g.numNeurons;
        std::vector<uint32_t> start(N + 1);
        HIP_TRY(hipMemcpy(start.data(), n.zeroStart, (size_t)(N + 1) * sizeof(uint32_t), hipMemcpyDeviceToHost));
        for(uint32_t b = 0; b < r->batch; b++) {
            uint32_t count = 0;
            HIP_TRY(hipMemcpy(&count, n.shadowCnt + (size_t)parity * r->batch + b, sizeof(uint32_t), hipMemcpyDeviceToHost));
            if(count == 0) { continue; }
            std::vector<uint32_t> spikes(count);
            HIP_TRY(hipMemcpy(spikes.data(), n.shadowSpk + ((size_t)parity * r->batch + b) * N, (size_t)count * sizeof(uint32_t), hipMemcpyDeviceToHost));
            for(uint32_t i : spikes) {
                const uint32_t len = start[i + 1] - start[i];
                if(len == 0) { continue; }
                std::vector<ZeroDelayEntry> entries(len);
                HIP_TRY(hipMemcpy(entries.data(), n.zeroEntries + start[i], (size_t)len * sizeof(ZeroDelayEntry), hipMemcpyDeviceToHost));
                for(const auto &e : entries) {
                    const uint32_t slot = (uint32_t)((r->epoch + 1) % e.maxDenDelay);      // the slot the coming step reads
                    out[{e.weight, b}] = e.ringElem + ((size_t)b * e.maxDenDelay + slot) * e.numTrgNeurons;
                }
            }
        }
    }
    return GENNMI_OK;
}

// Segment boundaries of the tile path for one projection; rows that are not sorted by target are reported through *unsorted
static int buildTileOffsets(const gennmi_presynaptic_update_group_t &g, uint16_t *dOff, uint32_t tileSize, uint32_t numTiles, uint32_t *unsorted)
{
    uint32_t *dFlag = nullptr;
    HIP_TRY(hipMalloc(&dFlag, sizeof(uint32_t)));
    HIP_TRY(hipMemset(dFlag, 0, sizeof(uint32_t)));
    tileOffsetKernel<<<dim3((g.numSrcNeurons + BLOCK - 1) / BLOCK), dim3(BLOCK), 0, 0>>>(
        g.numSrcNeurons, g.rowStride, g.rowLength, g.ind, tileSize, numTiles, dOff, dFlag);
    HIP_TRY(hipGetLastError());
    HIP_TRY(hipMemcpy(unsorted, dFlag, sizeof(uint32_t), hipMemcpyDeviceToHost));
    HIP_TRY(hipFree(dFlag));
    return GENNMI_OK;
}

// Ordered accumulation: a column view of every SPARSE projection it covers (engine-private: the user's own colLength /
// remap exist for plastic projections only) and one bitmap per distinct spike queue.  Called at finalise and again
// whenever the connectivity has been rewritten.
static int buildOrderedViews(gennmi_runner *r)
{
    for(void *q : r->orderedOwned) { hipFree(q); }
    r->orderedOwned.clear();
    r->orderedGroups.clear(); r->orderedPre.clear(); r->orderedSources.clear();
    if(r->dOrderedSources) { HIP_TRY(hipFree(r->dOrderedSources)); r->dOrderedSources = nullptr; }
    if(r->dOrderedBitmaps) { HIP_TRY(hipFree(r->dOrderedBitmaps)); r->dOrderedBitmaps = nullptr; }
    std::vector<size_t> bitmapOffset;       // of every source, in words
    size_t words = 0;
    for(size_t k = 0; k < r->pre.size(); k++) {
        auto &p = r->pre[k];
        const auto &g = p.g;
        const bool covered = g.matrix == GENNMI_MATRIX_SPARSE && (g.wum == GENNMI_WUM_STATIC_PULSE || g.wum == GENNMI_WUM_STATIC_PULSE_DENDRITIC_DELAY
                                                                  || g.wum == GENNMI_WUM_STDP_TRACE || g.wum == GENNMI_WUM_STDP);
        p.ordered = covered ? 1u : 0u;
        if(!covered) { continue; }
        if(g.maxDenDelay > ORDERED_MAX_SLOT_REGS * WAVE) { return fail(GENNMI_EUNSUPPORTED, "ordered accumulation: dendritic-delay rings of more than 256 slots"); }
        if((uint64_t)g.numSrcNeurons * g.rowStride > 0xFFFFFFFFull) { return fail(GENNMI_EUNSUPPORTED, "ordered accumulation: synapse index exceeds 32 bits (the column view holds 32-bit ids)"); }
        uint32_t maxLen = 0;
        { const int rc = gennmi_max_col_length(g.numSrcNeurons, g.numTrgNeurons, g.rowStride, g.rowLength, g.ind, &maxLen); if(rc) { return rc; } }
        OrderedGroupDev o{};
        o.g = g;
        o.colStride = std::max(1u, maxLen);
        uint32_t *colLength = nullptr, *remap = nullptr;
        HIP_TRY(hipMalloc(&colLength, (size_t)g.numTrgNeurons * sizeof(uint32_t)));
        r->orderedOwned.push_back(colLength);
        HIP_TRY(hipMalloc(&remap, (size_t)g.numTrgNeurons * o.colStride * sizeof(uint32_t)));
        r->orderedOwned.push_back(remap);
        { const int rc = gennmi_build_remap(g.numSrcNeurons, g.numTrgNeurons, g.rowStride, o.colStride, g.rowLength, g.ind, colLength, remap); if(rc) { return rc; } }
        o.colLength = colLength; o.remap = remap;
        // the queue this projection reads: shared with every other projection that reads the same slot of the same queue
        size_t src = r->orderedSources.size();
        for(size_t q = 0; q < r->orderedSources.size(); q++) {
            const auto &c = r->orderedSources[q];
            if(c.srcSpk == g.srcSpk && c.srcSpkCnt == g.srcSpkCnt && c.numSrcDelaySlots == g.numSrcDelaySlots && c.axonalDelaySteps == g.axonalDelaySteps) { src = q; }
        }
        if(src == r->orderedSources.size()) {
            OrderedSourceDev c{};
            c.srcSpk = g.srcSpk; c.srcSpkCnt = g.srcSpkCnt; c.numSrcNeurons = g.numSrcNeurons; c.words = (g.numSrcNeurons + 31) / 32;
            c.numSrcDelaySlots = g.numSrcDelaySlots; c.axonalDelaySteps = g.axonalDelaySteps;
            c.numBlocks = std::max(1u, std::min(64u, (g.numSrcNeurons + 16 * BLOCK - 1) / (16 * BLOCK)));
            bitmapOffset.push_back(words);
            words += (size_t)c.words * r->batch;
            r->orderedSources.push_back(c);
        }
        o.words = r->orderedSources[src].words;
        o.bitmap = reinterpret_cast<const uint32_t*>(bitmapOffset[src]);        // offset for now, pointer below
        r->orderedGroups.push_back(o);
        r->orderedPre.push_back(k);
    }
    r->scatterNeeded = false;
    for(const auto &p : r->pre) { r->scatterNeeded = r->scatterNeeded || !p.ordered; }
    if(r->orderedGroups.empty()) { return GENNMI_OK; }
    HIP_TRY(hipMalloc(&r->dOrderedBitmaps, words * sizeof(uint32_t)));
    HIP_TRY(hipMemset(r->dOrderedBitmaps, 0, words * sizeof(uint32_t)));
    r->orderedBitmapWords = words;
    for(auto &o : r->orderedGroups) { o.bitmap = r->dOrderedBitmaps + reinterpret_cast<uintptr_t>(o.bitmap); }
    std::vector<OrderedSourceDev> table;
    uint32_t block = 0;
    for(size_t q = 0; q < r->orderedSources.size(); q++) {
        auto &c = r->orderedSources[q];
        c.bitmap = r->dOrderedBitmaps + bitmapOffset[q];
        c.startBlock = block;
        block += c.numBlocks;
        for(uint32_t b = 0; b < c.numBlocks; b++) { table.push_back(c); }
    }
    r->orderedSourceBlocks = block;
    HIP_TRY(hipMalloc(&r->dOrderedSources, table.size() * sizeof(OrderedSourceDev)));
    HIP_TRY(hipMemcpy(r->dOrderedSources, table.data(), table.size() * sizeof(OrderedSourceDev), hipMemcpyHostToDevice));
    return GENNMI_OK;
}

static int buildTileRecords(const gennmi_runner *r, const gennmi_runner::RecordTable &t)
{
    const auto &g = r->pre[t.pre].g;
    const size_t count = (size_t)g.numSrcNeurons * t.numTiles;
    const dim3 grid((unsigned int)((count + BLOCK - 1) / BLOCK));
    if(t.lanes == 5) { tileRecordBuildKernel<5><<<grid, dim3(BLOCK), 0, 0>>>(g.numSrcNeurons, g.rowStride, g.ind, g.g, t.off, t.tileSize, t.numTiles, t.records, t.overflow); }
    else { tileRecordBuildKernel<10><<<grid, dim3(BLOCK), 0, 0>>>(g.numSrcNeurons, g.rowStride, g.ind, g.g, t.off, t.tileSize, t.numTiles, t.records, t.overflow); }
    HIP_TRY(hipGetLastError());
    HIP_TRY(hipDeviceSynchronize());
    return GENNMI_OK;
}

// Connectivity-derived tables follow the connectivity: when rowLength / ind / d of a projection have been written since
// the tables were built (a connectivity push after load), they are rebuilt before the next launch.
static int refreshTables(gennmi_runner *r)
{
    bool stale, recordsStale;
    {
        std::lock_guard<std::mutex> lock(g_runnersMutex);
        stale = r->tablesStale; recordsStale = r->recordsStale;
        r->tablesStale = false; r->recordsStale = false;
    }
    if(!stale && !recordsStale) { return GENNMI_OK; }
    HIP_TRY(hipStreamSynchronize(r->stream));
    if(!stale) {
        // only weights were written: the records hold copies of them
        for(const auto &t : r->recordTables) { const int rc = buildTileRecords(r, t); if(rc) { return rc; } }
        return GENNMI_OK;
    }
    for(const auto &t : r->tileTables) {
        uint32_t unsorted = 0;
        { const int rc = buildTileOffsets(r->pre[t.pre].g, t.off, t.tileSize, t.numTiles, &unsorted); if(rc) { return rc; } }
        if(unsorted) {
            return fail(GENNMI_ESTATE, "connectivity written after load leaves the rows of a projection no longer sorted by target, which its launch plan relies on; "
                                       "sort the rows or set GENNMI_TILE_FLOATS=0 before the runner is finalised");
        }
    }
    for(const auto &t : r->recordTables) { const int rc = buildTileRecords(r, t); if(rc) { return rc; } }
    if(r->fusedStep) {
        // The spikes of the last completed step have already had their zero-delay synapses delivered — by the old lists —
        // into the slot that is read next, and the coming step will skip every synapse that is zero-delay NOW.  Synapses of
        // those spikes that changed sides are put right here: newly zero-delay ones are added to that slot (exact), ones that
        // no longer are zero-delay are taken out again (a subtraction: the slot's sum is then right to rounding) and
        // delivered by the coming step like any other.
        std::map<std::pair<const float*, uint32_t>, float*> before, after;
        { const int rc = pendingZeroDelay(r, before); if(rc) { return rc; } }
        { const int rc = buildZeroDelayLists(r); if(rc) { return rc; } }
        { const int rc = pendingZeroDelay(r, after); if(rc) { return rc; } }
        std::vector<ZeroDelayCorrection> fix;
        for(const auto &e : after) { if(!before.count(e.first)) { fix.push_back({e.second, e.first.first, 1.0f, 0u}); } }
        for(const auto &e : before) { if(!after.count(e.first)) { fix.push_back({e.second, e.first.first, -1.0f, 0u}); } }
        if(!fix.empty()) {
            ZeroDelayCorrection *dFix = nullptr;
            HIP_TRY(hipMalloc(&dFix, fix.size() * sizeof(ZeroDelayCorrection)));
            HIP_TRY(hipMemcpy(dFix, fix.data(), fix.size() * sizeof(ZeroDelayCorrection), hipMemcpyHostToDevice));
            zeroDelayCorrectionKernel<<<dim3((unsigned int)((fix.size() + BLOCK - 1) / BLOCK)), dim3(BLOCK), 0, 0>>>(dFix, (uint32_t)fix.size());
            HIP_TRY(hipGetLastError());
            HIP_TRY(hipDeviceSynchronize());
            HIP_TRY(hipFree(dFix));
        }
        // the per-block descriptor tables carry the lists' addresses: same layout, new contents
        std::vector<NeuronGroupDev> neuronTable;
        for(const auto &g : r->neuron) { for(uint32_t b = 0; b < g.numBlocks; b++) { neuronTable.push_back(g); } }
        HIP_TRY(hipMemcpy(r->dNeuron, neuronTable.data(), neuronTable.size() * sizeof(NeuronGroupDev), hipMemcpyHostToDevice));
        std::vector<PreGroupDev> preTable;
        for(const auto &g : r->pre) { for(uint32_t b = 0; b < g.numBlocks; b++) { preTable.push_back(g); } }
        HIP_TRY(hipMemcpy(r->dPre, preTable.data(), preTable.size() * sizeof(PreGroupDev), hipMemcpyHostToDevice));
    }
    if(r->ordered) {
        // the gather kernels receive their column views by value, so a captured step graph holds the addresses of the views
        // just freed: it is captured again on the next replay
        if(r->graphExec) { HIP_TRY(hipGraphExecDestroy(r->graphExec)); r->graphExec = nullptr; r->graphSteps = 0; }
        const int rc = buildOrderedViews(r);
        if(rc) { return rc; }
    }
    return GENNMI_OK;
}

int gennmi_runner_set_ordered(gennmi_runner *r, int enabled)
{
    if(!r) { return fail(GENNMI_EINVAL, "runner_set_ordered: null runner"); }
    if(r->finalised) { return fail(GENNMI_ESTATE, "runner_set_ordered: the accumulation mode is fixed when the runner is finalised"); }
    r->ordered = (enabled != 0);
    return GENNMI_OK;
}

int gennmi_runner_finalise(gennmi_runner *r)
{
    if(!r) { return fail(GENNMI_EINVAL, "runner_finalise: null runner"); }
    if(r->finalised) { return fail(GENNMI_ESTATE, "runner_finalise: called twice"); }
    if(r->neuron.empty()) { return fail(GENNMI_EINVAL, "runner_finalise: no neuron groups"); }
    int device = 0;
    HIP_TRY(hipGetDevice(&device));
    hipDeviceProp_t prop;
    HIP_TRY(hipGetDeviceProperties(&prop, device));
    const uint32_t numCU = (uint32_t)prop.multiProcessorCount;

    if(const char *envOrdered = getenv("GENNMI_ORDERED")) { r->ordered = r->ordered || atoi(envOrdered) != 0; }
    // a projection's view of its source's delay slots must be the source's own
    for(const auto &p : r->pre) {
        for(const auto &n : r->neuron) {
            if(n.g.spk == p.g.srcSpk && std::max(1u, n.g.numDelaySlots) != std::max(1u, p.g.numSrcDelaySlots)) {
                return fail(GENNMI_EINVAL, "runner_finalise: a projection and its source population disagree on the number of delay slots");
            }
        }
    }
    // ---- plastic projections: pair the postsynaptic pass of each with its presynaptic half (LearnPostDev), so that every
    // synapse has one writer per step and the passes can share a launch.  Needs the spikes of the last neuron update of both
    // populations as bitmaps, which their neuron updates keep.  GENNMI_PAIRED_LEARN=0 leaves the passes as two launches in a row.
    {
        const char *envPaired = getenv("GENNMI_PAIRED_LEARN");
        const bool pairing = !r->ordered && !(envPaired && atoi(envPaired) == 0);
        auto populationOf = [r](const uint32_t *queue, uint32_t numNeurons) -> NeuronGroupDev*
        {
            for(auto &n : r->neuron) {
                bool feeds = (n.g.spk == queue);
                for(uint32_t q = 0; q < n.g.numExtraSpk; q++) { feeds = feeds || (n.g.extraSpk[q] == queue); }
                if(feeds && n.g.numNeurons == numNeurons) { return &n; }
            }
            return nullptr;
        };
        auto bitmapOf = [r](NeuronGroupDev *n) -> hipError_t
        {
            if(n->spikeBitmap) { return hipSuccess; }
            const size_t bytes = (size_t)r->batch * ((n->g.numNeurons + 31) / 32) * sizeof(uint32_t);
            hipError_t e = hipMalloc((void**)&n->spikeBitmap, bytes);
            if(e != hipSuccess) { return e; }
            r->owned.push_back(n->spikeBitmap);
            return hipMemset(n->spikeBitmap, 0, bytes);
        };
        r->combinePost = pairing && !r->post.empty();
        for(auto &p : r->post) {
            PreGroupDev *partner = nullptr;
            for(auto &q : r->pre) {
                if(q.g.g == p.g.g && (q.g.wum == GENNMI_WUM_STDP_TRACE || q.g.wum == GENNMI_WUM_STDP) && q.g.matrix == GENNMI_MATRIX_SPARSE
                   && q.g.numSrcDelaySlots <= 1 && q.g.numSrcNeurons == p.g.numSrcNeurons && q.g.numTrgNeurons == p.g.numTrgNeurons) { partner = &q; }
            }
            NeuronGroupDev *src = partner ? populationOf(partner->g.srcSpk, p.g.numSrcNeurons) : nullptr;
            NeuronGroupDev *trg = populationOf(p.g.trgSpk, p.g.numTrgNeurons);
            if(!pairing || !partner || !src || !trg || std::max(1u, src->g.numDelaySlots) > 1 || std::max(1u, trg->g.numDelaySlots) > 1) { r->combinePost = false; continue; }
            HIP_TRY(bitmapOf(src));
            HIP_TRY(bitmapOf(trg));
            partner->learn.srcST = p.g.srcST; partner->learn.preTrace = p.g.preTrace; partner->learn.trgBitmap = trg->spikeBitmap;
            partner->learn.aPlus = p.g.aPlus; partner->learn.tauPlus = p.g.tauPlus; partner->learn.enabled = 1;
            p.srcBitmap = src->spikeBitmap;
        }
    }
    // Large networks of plain groups take the several-neurons-per-lane kernel: what counts is the number of rounds of
    // resident work-groups a launch needs (numCU x 8 work-groups of 256 lanes are resident at a time).
    {
        unsigned long long lanes = 0;
        bool plain = r->post.empty();
        for(const auto &n : r->neuron) {
            const auto &g = n.g;
            lanes += (unsigned long long)g.numNeurons * r->batch;
            for(uint32_t c = 0; c < g.numCS; c++) { plain = plain && g.cs[c].kind != GENNMI_CS_POISSON_EXP; }
            plain = plain && g.numPSM <= BULK_MAX_PSM && g.numCS <= BULK_MAX_CS && !g.preTrace && !g.postTrace && !g.sT && g.numExtraSpk == 0
                    && g.numDelaySlots <= 1 && g.numSpkEvent == 0 && g.numPreOutput == 0;
        }
        // measured: four per lane from one round of work-groups up (10^6 Izhikevich neurons: 20.1 us with one, 18.0 with two,
        // 16.4 with four), eight beyond five rounds (3.1 x 10^6 lanes of the batched convolution layer: 57 / 38 / 29 / 24 us
        // with one / two / four / eight); GENNMI_NEURON_BULK = 0 (never), 2, 4 or 8 forces the choice
        const unsigned long long round = 1ull * numCU * 8 * BLOCK;
        uint32_t perLane = (lanes <= round) ? 1u : (2 * lanes <= 5 * round) ? 4u : 8u;
        if(const char *envBulk = getenv("GENNMI_NEURON_BULK")) {
            const int v = atoi(envBulk);
            perLane = (v == 2 || v == 4 || v == 8) ? (uint32_t)v : (v == 1) ? 4u : 1u;
        }
        r->neuronsPerLane = plain ? perLane : 1u;
        r->plainGroups = plain;
    }
    const uint32_t neuronsPerBlock = BLOCK * r->neuronsPerLane;
    uint32_t block = 0;
    for(auto &n : r->neuron) {
        n.startBlock = block;
        n.numBlocks = (n.g.numNeurons + neuronsPerBlock - 1) / neuronsPerBlock;
        block += n.numBlocks;
    }
    r->neuronBlocks = block;


    // DENSE / BITMASK projections: one lane per postsynaptic neuron; a group owns its outPost unless another dense or
    // bitmask group adds to the same one (sparse groups have finished by the time this kernel starts)
    block = 0;
    for(auto &d : r->dense) {
        const uint32_t columnBlocks = (d.g.numTrgNeurons + BLOCK - 1) / BLOCK;
        // enough blocks to cover the chip a few times when a step carries many spikes
        d.slices = std::max(1u, std::min({64u, (4u * numCU + columnBlocks - 1) / columnBlocks, (d.g.numSrcNeurons + DENSE_SPIKES_PER_SLICE - 1) / DENSE_SPIKES_PER_SLICE}));
        d.startBlock = block;
        d.numBlocks = columnBlocks * d.slices;
        block += d.numBlocks;
        d.exclusive = 1;
        for(const auto &o : r->dense) { if(&o != &d && o.g.outPost == d.g.outPost) { d.exclusive = 0; } }
    }
    r->denseBlocks = block;

    // PROCEDURAL projections: a wavefront per spike; enough wavefronts for ~1.5 % of the source population firing at once
    block = 0;
    for(auto &p : r->proc) {
        const uint32_t wantWaves = std::max(8u, p.g.numSrcNeurons / 64);
        p.startBlock = block;
        p.numBlocks = std::max(1u, std::min((wantWaves + (BLOCK / WAVE) - 1) / (BLOCK / WAVE), 8u * numCU / std::max<uint32_t>(1, (uint32_t)r->proc.size())));
        block += p.numBlocks;
    }
    r->procBlocks = block;

    // One descriptor copy per block, indexed by blockIdx.x: a block finds everything it needs with a
    // single round of scalar loads (the reference bisects a start-ID table and then loads the merged
    // struct, backendSIMT.h:244-323 — two to four dependent loads before any work starts).
    auto uploadPerBlock = [](const auto &groups, uint32_t totalBlocks, auto **dTable) -> hipError_t {
        using T = typename std::remove_reference<decltype(groups[0])>::type;
        std::vector<typename std::remove_const<T>::type> table;
        table.reserve(totalBlocks);
        for(const auto &g : groups) { for(uint32_t b = 0; b < g.numBlocks; b++) { table.push_back(g); } }
        if(table.empty()) { *dTable = nullptr; return hipSuccess; }
        hipError_t e = hipMalloc(dTable, table.size() * sizeof(table[0]));
        if(e != hipSuccess) { return e; }
        return hipMemcpy(*dTable, table.data(), table.size() * sizeof(table[0]), hipMemcpyHostToDevice);
    };
    // ---- tile path for delay-free SPARSE projections (static or trace-STDP weights) whose rows are sorted by target
    {
        const char *envTile = getenv("GENNMI_TILE_FLOATS");
        // (ordered accumulation gathers SPARSE projections itself: no tile paths then)
        const uint32_t tileFloats = r->ordered ? 0u : envTile ? (uint32_t)std::max(0, atoi(envTile)) : 16384u;
        const char *envThreads = getenv("GENNMI_TILE_THREADS");
        r->tileThreads = envThreads ? (uint32_t)std::min(1024, std::max(64, atoi(envThreads))) : (tileFloats > 16384 ? 1024u : (tileFloats > 8192 ? 512u : (uint32_t)BLOCK));
        std::vector<TileGroupDev> tiles, tileGroups;
        std::vector<ConvTileDev> convTiles;
        for(auto &p : r->pre) {
            p.workPerSpike = (p.g.matrix == GENNMI_MATRIX_SPARSE) ? p.g.rowStride : (uint32_t)(p.g.conv[0] * p.g.conv[1] * p.g.conv[7]);
            if(p.g.numSrcDelaySlots > 1) { continue; }       // the tile kernels read the queue without delay slots
            if(tileFloats != 0 && p.g.matrix == GENNMI_MATRIX_TOEPLITZ_CONV2D && r->pre.size() == 1
               && p.g.conv[0] < 1024 && p.g.conv[1] < 1024 && p.g.conv[7] < 1024
               && p.g.conv[2] < 1024 && p.g.conv[3] < 1024 && p.g.conv[4] < 1024) {        // rows, columns and channels are packed 10 bits each
                const int32_t *c = p.g.conv;
                // the matrix cores take the layer when its source's neuron update can keep a spike bitmap and a block's patch
                // and the kernel fit in LDS (GENNMI_CONV_MFMA=0: the event-driven tile kernel below)
                {
                    const char *envMfma = getenv("GENNMI_CONV_MFMA");
                    NeuronGroupDev *src = nullptr;
                    for(auto &n : r->neuron) { if(n.g.spk == p.g.srcSpk && n.g.numNeurons == p.g.numSrcNeurons) { src = &n; } }
                    if(!(envMfma && atoi(envMfma) == 0) && src) {
                        ConvMfmaDev m{};
                        m.g = p.g; m.convBH = p.convBH; m.convBW = p.convBW;
                        const uint32_t K = (uint32_t)(c[0] * c[1] * c[4]);
                        m.kernPitch = ((uint32_t)c[7] + 31) / 32 * 32;
                        if(m.kernPitch % 64 == 0) { m.kernPitch += 32; }         // the two halves of a wavefront read consecutive rows
                        m.patchPitch = ((uint32_t)c[6] + 31) / 32 * 32 + (uint32_t)c[1] - 1;
                        const size_t kernFloats = (size_t)2 * (((K + 1) / 2 + CONV_MFMA_STEPS - 1) / CONV_MFMA_STEPS) * CONV_MFMA_STEPS * m.kernPitch;       // whole chunks of steps
                        // as many output rows per block as give every compute unit one block, fewer if LDS says so
                        uint32_t rowsPerBlock = std::max(1u, std::min<uint32_t>((uint32_t)c[5], ((uint32_t)c[5] * r->batch) / numCU));
                        if(const char *envRows = getenv("GENNMI_CONV_ROWS")) { rowsPerBlock = std::max(1u, std::min<uint32_t>((uint32_t)c[5], (uint32_t)atoi(envRows))); }
                        size_t bytes = 0;
                        for(;; rowsPerBlock--) {
                            m.patchRows = rowsPerBlock + (uint32_t)c[0] - 1;
                            m.planePitch = (m.patchRows * m.patchPitch + 63) / 64 * 64 + 32;
                            bytes = ((size_t)c[4] * m.planePitch + kernFloats) * sizeof(float);
                            if(bytes <= 64 * 1024 || rowsPerBlock == 1) { break; }
                        }
                        if(bytes <= 64 * 1024) {
                            if(!src->spikeBitmap) {
                                const size_t bitmapBytes = (size_t)r->batch * ((src->g.numNeurons + 31) / 32) * sizeof(uint32_t);
                                HIP_TRY(hipMalloc((void**)&src->spikeBitmap, bitmapBytes));
                                r->owned.push_back(src->spikeBitmap);
                                HIP_TRY(hipMemset(src->spikeBitmap, 0, bitmapBytes));
                                r->bitmapsStale = true;          // the queue may already hold spikes
                            }
                            m.srcBitmap = src->spikeBitmap;
                            r->convSource = (size_t)(src - r->neuron.data());
                            m.rowsPerBlock = rowsPerBlock;
                            m.numBatches = r->batch;
                            p.tileThreshold = std::max(1u, p.g.numTrgNeurons / 4);
                            m.threshold = p.tileThreshold;
                            r->convMfma = m;
                            HIP_TRY(hipMalloc(&r->dConvMfma, sizeof(ConvMfmaDev)));
                            HIP_TRY(hipMemcpy(r->dConvMfma, &m, sizeof(ConvMfmaDev), hipMemcpyHostToDevice));
                            r->owned.push_back(r->dConvMfma);
                            r->convMfmaBlocks = ((uint32_t)c[5] + rowsPerBlock - 1) / rowsPerBlock;
                            r->convMfmaBytes = bytes;
                            if(bytes > 48 * 1024) {
                                HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void*>(presynapticConvMfmaKernel), hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes));
                            }
                            continue;
                        }
                    }
                }
                const size_t rowFloats = (size_t)c[6] * c[7];
                const size_t fixedFloats = (size_t)c[0] * c[1] * c[4] * c[7] + CONV_TILE_SPIKES;      // kernel weights + staged spikes
                const size_t budgetFloats = 60 * 1024 / sizeof(float);
                if(fixedFloats + rowFloats <= budgetFloats) {
                    // as many rows per block as fit in LDS, but enough blocks to cover the chip once
                    uint32_t rowsPerTile = (uint32_t)std::min<size_t>((budgetFloats - fixedFloats) / rowFloats, (size_t)c[5]);
                    // measured on the batched 64x64 layer (us per launch of both presynaptic kernels): 119 / 75 / 61 with 4 / 2 / 1
                    // blocks per compute unit — a spike concerns (rows + kh - 1) / rows tiles, so fewer, taller tiles do less
                    // redundant work
                    const char *envConvBlocks = getenv("GENNMI_CONV_TILE_BLOCKS_PER_CU");
                    const uint32_t convBlocksPerCU = envConvBlocks ? (uint32_t)std::max(1, atoi(envConvBlocks)) : 1u;
                    const uint32_t wantBlocks = std::max(1u, (convBlocksPerCU * numCU) / r->batch);
                    rowsPerTile = std::max(1u, std::min(rowsPerTile, ((uint32_t)c[5] + wantBlocks - 1) / wantBlocks));
                    ConvTileDev t{};
                    t.g = p.g; t.convBH = p.convBH; t.convBW = p.convBW; t.rowsPerTile = rowsPerTile;
                    p.tileThreshold = std::max(1u, p.g.numTrgNeurons / 4);
                    t.threshold = p.tileThreshold;
                    for(uint32_t row0 = 0; row0 < (uint32_t)c[5]; row0 += rowsPerTile) { t.tileRow0 = row0; convTiles.push_back(t); }
                    r->convTileBytes = (fixedFloats + rowsPerTile * rowFloats) * sizeof(float);
                }
                continue;
            }
            if(tileFloats == 0 || p.g.matrix != GENNMI_MATRIX_SPARSE || p.g.rowStride > 65535
               || (p.g.wum != GENNMI_WUM_STATIC_PULSE && p.g.wum != GENNMI_WUM_STDP_TRACE && p.g.wum != GENNMI_WUM_STDP)) { continue; }
            const uint32_t tileSize = std::min(tileFloats, p.g.numTrgNeurons);
            const uint32_t numTiles = (p.g.numTrgNeurons + tileSize - 1) / tileSize;
            uint16_t *dOff = nullptr;
            HIP_TRY(hipMalloc(&dOff, (size_t)p.g.numSrcNeurons * (numTiles + 1) * sizeof(uint16_t)));
            r->owned.push_back(dOff);
            uint32_t unsorted = 0;
            { const int rc = buildTileOffsets(p.g, dOff, tileSize, numTiles, &unsorted); if(rc) { return rc; } }
            if(unsorted) { continue; }          // rows not sorted by target: the scatter kernel handles every step
            p.tileThreshold = std::max(1u, p.g.numTrgNeurons);
            r->tileTables.push_back({(size_t)(&p - r->pre.data()), dOff, tileSize, numTiles});
            const uint32_t avgSeg = std::max(1u, p.g.rowStride / numTiles);
            TileGroupDev t{};
            t.g = p.g; t.learn = p.learn; t.tileOff = dOff; t.numTiles = numTiles; t.tileSize = tileSize;
            const char *envLanes = getenv("GENNMI_TILE_LANES");
            t.lanes = envLanes ? std::min<uint32_t>(WAVE, pow2Ceil((uint32_t)std::max(1, atoi(envLanes)))) : std::min<uint32_t>(WAVE, pow2Ceil((avgSeg + 7) / 8));
            t.threshold = p.tileThreshold;
            // Short segments (a row spread over many tiles) are what the plain tile path reads worst: two short reads at
            // arbitrary offsets plus the boundary look-up per (spike, tile).  Static projections whose segments fit a
            // record of 20 or 40 synapses get the record copy; GENNMI_TILE_RECORDS=0 keeps the rows only.
            const char *envRecords = getenv("GENNMI_TILE_RECORDS");
            const uint32_t segLen = (p.g.rowStride + numTiles - 1) / numTiles;
            if(!(envRecords && atoi(envRecords) == 0) && p.g.wum == GENNMI_WUM_STATIC_PULSE && segLen >= 6 && segLen <= 34 && tileSize <= 65536) {
                const uint32_t lanes = (segLen <= 17) ? 5u : 10u;
                const size_t bytes = (size_t)numTiles * p.g.numSrcNeurons * recordBytes(lanes);
                size_t freeBytes = 0, totalBytes = 0;
                HIP_TRY(hipMemGetInfo(&freeBytes, &totalBytes));
                if(bytes + (size_t(2) << 30) < freeBytes) {
                    uint8_t *records = nullptr;
                    HIP_TRY(hipMalloc(&records, bytes));
                    r->owned.push_back(records);
                    // overflow records where memory allows: segments are Poisson-like around rowStride / numTiles, so a
                    // sixth or so of them exceed a record sized for the mean
                    uint8_t *overflow = nullptr;
                    const size_t overflowBytes = (size_t)numTiles * p.g.numSrcNeurons * 64;
                    if(bytes + overflowBytes + (size_t(2) << 30) < freeBytes) {
                        HIP_TRY(hipMalloc(&overflow, overflowBytes));
                        r->owned.push_back(overflow);
                    }
                    const gennmi_runner::RecordTable table{(size_t)(&p - r->pre.data()), records, overflow, dOff, lanes, tileSize, numTiles};
                    { const int rc = buildTileRecords(r, table); if(rc) { return rc; } }
                    r->recordTables.push_back(table);
                    t.records = records; t.recLanes = lanes; t.overflow = overflow;
                }
            }
            tileGroups.push_back(t);
            r->tileFloats = std::max(r->tileFloats, tileSize);
        }
        if(!tileGroups.empty()) {
            // Every group gets a whole resident round of the chip (GENNMI_TILE_BLOCKS_PER_CU x 256 threads per compute
            // unit): activity is bursty, a burst in one projection should find all compute units, and the blocks of
            // groups whose step went to the scatter kernel leave after reading one counter.
            const char *envSplit = getenv("GENNMI_TILE_BLOCKS_PER_CU");
            const uint32_t blocksPerCUTile = envSplit ? (uint32_t)std::max(1, atoi(envSplit)) : 4u;
            const uint32_t budget = blocksPerCUTile * numCU * BLOCK / r->tileThreads;
            // ... several groups share two such rounds in proportion to their synapse counts: a launch's floor is the
            // dispatch of its blocks, and the quiet steps of a network with many projections should not pay for a round each
            const char *envPerSplit = getenv("GENNMI_TILE_SPIKES_PER_SPLIT");
            const uint32_t spikesPerSplit = envPerSplit ? (uint32_t)std::max(1, atoi(envPerSplit)) : 4096u;
            double totalWeight = 0.0;
            for(const auto &t : tileGroups) { totalWeight += (double)t.g.numSrcNeurons * t.g.rowStride; }
            for(auto &t : tileGroups) {
                const double share = (tileGroups.size() == 1) ? 1.0 : 2.0 * ((double)t.g.numSrcNeurons * t.g.rowStride) / totalWeight;
                const uint32_t groupBudget = std::max(t.numTiles, (uint32_t)(share * budget));
                const uint32_t numSplits = std::max(1u, std::min(256u, groupBudget / t.numTiles));
                t.numSplits = numSplits;
                t.spikesPerSplit = spikesPerSplit;
                for(uint32_t tile = 0; tile < t.numTiles; tile++) {
                    for(uint32_t split = 0; split < numSplits; split++) { t.tile = tile; t.split = split; tiles.push_back(t); }
                }
            }
        }
        if(!convTiles.empty()) {
            HIP_TRY(hipMalloc(&r->dConvTile, convTiles.size() * sizeof(ConvTileDev)));
            HIP_TRY(hipMemcpy(r->dConvTile, convTiles.data(), convTiles.size() * sizeof(ConvTileDev), hipMemcpyHostToDevice));
            r->convTileBlocks = (uint32_t)convTiles.size();
            if(r->convTileBytes > 48 * 1024) {
                HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void*>(presynapticConvTileKernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                            (int)r->convTileBytes));
            }
        }
        if(!tiles.empty()) {
            HIP_TRY(hipMalloc(&r->dTile, tiles.size() * sizeof(TileGroupDev)));
            HIP_TRY(hipMemcpy(r->dTile, tiles.data(), tiles.size() * sizeof(TileGroupDev), hipMemcpyHostToDevice));
            r->tileBlocks = (uint32_t)tiles.size();
            if((size_t)r->tileFloats * sizeof(float) > 48 * 1024) {
                HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void*>(presynapticTileKernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                            (int)(r->tileFloats * sizeof(float))));
            }
        }
    }

    // Presynaptic launch geometry.  The number of spikes is only known on the device, so every
    // group gets a fixed number of blocks and deals its (spike, chunk) work items round-robin to their
    // sub-groups.  A group wants enough sub-groups for ~1.5 % of its source population firing in one step; when
    // the groups together want more than the budget, it is shared in proportion (work per step scales with
    // source size x row length, whatever the rates turn out to be).
    // Scatter, tile and postsynaptic blocks may share a launch (synapseCombinedKernel), so all three use the tile path's
    // block size where there is one; budgets are in blocks of 256 threads and converted.
    block = 0;
    const uint32_t synThreads = r->tileBlocks ? r->tileThreads : (uint32_t)BLOCK;
    r->synapseThreads = synThreads;
    const char *envBudget = getenv("GENNMI_PRESYN_BLOCKS_PER_CU");
    // (2, not more: measured with 4 / 2 / 1 — 100 k-neuron plastic network 23.8 / 22.6 / 22.6 us per step, 10^6-neuron fan-out network
    // 45.6 / 44.0 / 44.8, microcircuit stepped launch by launch 11.8 / 11.4 / 12.2: a quiet step pays for every block it dispatches)
    const uint32_t blocksPerCU = envBudget ? std::max(1, atoi(envBudget)) : 2u;
    // the launch has one grid row per batch, so the budget is per batch (at least one block per compute unit in all)
    const uint64_t budget = std::max<uint64_t>((numCU + r->batch - 1) / r->batch, (uint64_t)numCU * blocksPerCU * BLOCK / synThreads / r->batch);
    std::vector<uint64_t> wantBlocks;
    for(auto &p : r->pre) {
        const uint32_t rowLen = (p.g.matrix == GENNMI_MATRIX_SPARSE) ? p.g.rowStride : (uint32_t)(p.g.conv[0] * p.g.conv[1] * p.g.conv[7]);
        uint32_t W;
        if(p.g.span == GENNMI_SPAN_PRE) { W = std::min(64u, pow2Ceil(std::max(1u, p.g.numThreadsPerSpike))); }
        else if(p.g.span == GENNMI_SPAN_POST) { W = WAVE; }
        else { W = std::min<uint32_t>(WAVE, std::max(4u, pow2Ceil((rowLen + 3) / 4))); }
        p.lanesPerSpike = W;
        p.vec4 = (p.g.matrix == GENNMI_MATRIX_SPARSE && p.g.wum != GENNMI_WUM_STDP_TRACE && p.g.wum != GENNMI_WUM_STDP && (p.g.rowStride % 4) == 0
                  && (reinterpret_cast<uintptr_t>(p.g.ind) % 16) == 0 && (reinterpret_cast<uintptr_t>(p.g.g) % 16) == 0
                  && (p.g.wum != GENNMI_WUM_STATIC_PULSE_DENDRITIC_DELAY || (reinterpret_cast<uintptr_t>(p.g.d) % 4) == 0)
                  && W >= 16) ? 1u : 0u;
        const uint32_t span = W * (p.vec4 ? 4u : 1u);
        const uint64_t chunksPerRow = (rowLen + span - 1) / span;
        const uint64_t wantSubGroups = std::max<uint64_t>(8, ((uint64_t)p.g.numSrcNeurons * chunksPerRow) / 64);
        wantBlocks.push_back(std::min<uint64_t>((wantSubGroups * W + synThreads - 1) / synThreads, budget));
    }
    uint64_t wantTotal = 0;
    for(uint64_t w : wantBlocks) { wantTotal += w; }
    for(size_t k = 0; k < r->pre.size(); k++) {
        auto &p = r->pre[k];
        const uint64_t blocks = (wantTotal <= budget) ? wantBlocks[k] : (wantBlocks[k] * budget + wantTotal - 1) / wantTotal;
        p.startBlock = block;
        p.numBlocks = (uint32_t)std::max<uint64_t>(1, blocks);
        block += p.numBlocks;
    }
    r->preBlocks = block;

    block = 0;
    for(auto &p : r->post) {
        p.lanesPerSpike = std::min<uint32_t>(WAVE, std::max(4u, pow2Ceil((p.g.colStride + 3) / 4)));
        const uint64_t wantSubGroups = std::max<uint64_t>(8, p.g.numTrgNeurons / 16);
        const char *envPost = getenv("GENNMI_POST_BLOCKS_PER_CU");
        const uint32_t postPerCU = envPost ? (uint32_t)std::max(1, atoi(envPost)) : 4u;
        const uint32_t cap = std::max(1u, (numCU * postPerCU * BLOCK / synThreads) / (uint32_t)r->post.size());
        p.startBlock = block;
        p.numBlocks = std::max(1u, (uint32_t)std::min<uint64_t>((wantSubGroups * p.lanesPerSpike + synThreads - 1) / synThreads, cap));
        block += p.numBlocks;
    }
    r->postBlocks = block;

    // ---- single-launch step: possible when every projection is a SPARSE dendritic-delay one with ring depth >= 2
    // and nothing is plastic
    bool anyEvents = false;
    for(const auto &n : r->neuron) { anyEvents = anyEvents || n.g.numSpkEvent != 0; }
    const char *envFused = getenv("GENNMI_FUSED_STEP");
    bool eligible = !r->ordered && !(envFused && atoi(envFused) == 0) && !r->pre.empty() && r->post.empty() && r->dense.empty() && r->proc.empty() && !anyEvents && r->neuronsPerLane == 1;
    for(const auto &p : r->pre) {
        eligible = eligible && p.g.matrix == GENNMI_MATRIX_SPARSE && p.g.wum == GENNMI_WUM_STATIC_PULSE_DENDRITIC_DELAY
                   && p.g.maxDenDelay >= 2 && p.g.numSrcDelaySlots <= 1;
        bool found = false;
        for(const auto &n : r->neuron) { found = found || (n.g.spk == p.g.srcSpk && n.g.numNeurons == p.g.numSrcNeurons); }
        eligible = eligible && found;
    }
    if(eligible) {
        const int rc = buildZeroDelayLists(r);
        if(rc) { return rc; }
        r->fusedStep = true;
    }
    // ---- dense-activity path of learnPost: the neuron update of the target population keeps a bitmap of the step's
    // spikes, and steps in which at least 1/8 of the targets fired walk the rows
    for(auto &p : r->post) {
        const uint32_t words = (p.g.numTrgNeurons + 31) / 32;
        if(!p.g.rowLength || !p.g.ind || words * sizeof(uint32_t) > 60 * 1024) { continue; }
        for(auto &n : r->neuron) {
            bool feeds = (n.g.spk == p.g.trgSpk);
            for(uint32_t q = 0; q < n.g.numExtraSpk; q++) { feeds = feeds || (n.g.extraSpk[q] == p.g.trgSpk); }
            if(!feeds || n.g.numNeurons != p.g.numTrgNeurons) { continue; }
            if(!n.spikeBitmap) {
                HIP_TRY(hipMalloc((void**)&n.spikeBitmap, (size_t)r->batch * words * sizeof(uint32_t)));
                HIP_TRY(hipMemset(n.spikeBitmap, 0, (size_t)r->batch * words * sizeof(uint32_t)));
                r->owned.push_back(n.spikeBitmap);
            }
            p.spikeBitmap = n.spikeBitmap;
            const char *envDiv = getenv("GENNMI_POST_DENSE_DIVISOR");      // rows are walked from numTrg / divisor spikes on (0: never)
            const uint32_t divisor = envDiv ? (uint32_t)std::max(0, atoi(envDiv)) : 8u;
            p.denseThreshold = divisor ? std::max(1u, p.g.numTrgNeurons / divisor) : 0u;
            r->postLdsBytes = std::max<uint32_t>(r->postLdsBytes, words * sizeof(uint32_t));
        }
    }
    if(r->postLdsBytes > 48 * 1024) {
        HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void*>(postsynapticUpdateKernel), hipFuncAttributeMaxDynamicSharedMemorySize, (int)r->postLdsBytes));
    }
    // ---- one launch for scatter path, tile path and paired postsynaptic passes (GENNMI_COMBINED=0: a launch each)
    {
        const char *envCombined = getenv("GENNMI_COMBINED");
        r->combineSynapses = !r->ordered && !(envCombined && atoi(envCombined) == 0) && (r->tileBlocks != 0 || r->combinePost);
        r->combinedLdsBytes = std::max<size_t>(r->tileBlocks ? (size_t)r->tileFloats * sizeof(float) : 0, r->combinePost ? r->postLdsBytes : 0);
        if(r->combineSynapses && r->combinedLdsBytes > 48 * 1024) {
            HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void*>(synapseCombinedKernel), hipFuncAttributeMaxDynamicSharedMemorySize, (int)r->combinedLdsBytes));
        }
    }
    if(r->ordered && r->batch != 1 && !r->post.empty()) { return fail(GENNMI_EUNSUPPORTED, "runner_finalise: ordered accumulation of plastic projections needs batch size 1"); }
    // spike sources: per-neuron copy of the next spike time, built before the first step and again after writes to the arrays
    for(auto &n : r->neuron) {
        if(n.g.model != GENNMI_NEURON_SPIKE_SOURCE_ARRAY) { continue; }
        // spikeTimes comes without a length: everything up to the end of its allocation counts as the array
        hipDeviceptr_t base = nullptr; size_t size = 0;
        HIP_TRY(hipMemGetAddressRange(&base, &size, const_cast<float*>(n.g.spikeTimes)));
        n.spikeTimesBytes = (reinterpret_cast<uintptr_t>(base) + size) - reinterpret_cast<uintptr_t>(n.g.spikeTimes);
        HIP_TRY(hipMalloc(&n.nextSpikeTime, (size_t)r->batch * n.g.numNeurons * sizeof(float)));
        r->owned.push_back(n.nextSpikeTime);
        r->sourcesStale = true;
    }
    // look-back area of the spike-like event queues: per event slot, per-block counts then per-group totals
    if(anyEvents) {
        const size_t count = (size_t)GENNMI_MAX_SPK_EVENT * 2 * r->neuronBlocks * r->batch;
        unsigned long long *area = nullptr;
        HIP_TRY(hipMalloc(&area, count * sizeof(unsigned long long)));
        r->owned.push_back(area);
        HIP_TRY(hipMemset(area, 0, count * sizeof(unsigned long long)));
        for(auto &n : r->neuron) { n.aggEvent = area; }
    }
    if(r->ordered) { const int rc = buildOrderedViews(r); if(rc) { return rc; } }
    // ---- a convolutional layer's whole step in one launch: the layer on the matrix cores is the model's only projection and its
    // target is a plain population whose only input it is (GENNMI_CONV_STEP=0: the layer's kernel, then the neuron kernel)
    if(r->convMfmaBlocks && !r->ordered) {
        const char *envStep = getenv("GENNMI_CONV_STEP");
        ConvMfmaDev &m = r->convMfma;
        const uint32_t ow = (uint32_t)m.g.conv[6], oc = (uint32_t)m.g.conv[7];
        NeuronGroupDev *target = nullptr;
        for(auto &n : r->neuron) {
            if(n.g.numPSM == 1 && n.g.psm[0].outPost == m.g.outPost && n.g.numNeurons == m.g.numTrgNeurons) { target = &n; }
        }
        NeuronGroupDev *src = &r->neuron[r->convSource];
        m.spikeWords = (m.rowsPerBlock * ow * oc + 31) / 32 + 1;
        const size_t bytes = r->convMfmaBytes + (size_t)m.spikeWords * sizeof(uint32_t);
        bool eligible = !(envStep && atoi(envStep) == 0) && r->plainGroups && target && target != src && bytes <= 64 * 1024 && (m.rowsPerBlock * ow * oc) % 32 == 0;
        if(eligible) {
            const auto &g = target->g;
            eligible = (g.model == GENNMI_NEURON_LIF || g.model == GENNMI_NEURON_IZHIKEVICH) && g.psm[0].maxDenDelay == 0
                       && (g.psm[0].kind == GENNMI_PSM_EXPCURR || g.psm[0].kind == GENNMI_PSM_DELTACURR)
                       && (g.numCS == 0 || (g.numCS == 1 && g.cs[0].kind == GENNMI_CS_DC)) && !g.preTrace && !g.postTrace && !g.sT && g.numExtraSpk == 0
                       && g.numDelaySlots <= 1 && g.numSpkEvent == 0 && g.numPreOutput == 0 && !target->spikeBitmap && !target->shadowSpk;
        }
        if(eligible) {
            // the source's spike bitmap twice: the layer reads last step's copy while the source's blocks of the same launch write this step's
            const size_t words = (size_t)r->batch * ((src->g.numNeurons + 31) / 32);
            uint32_t *both = nullptr;
            HIP_TRY(hipMalloc((void**)&both, 2 * words * sizeof(uint32_t)));
            r->owned.push_back(both);
            HIP_TRY(hipMemset(both, 0, 2 * words * sizeof(uint32_t)));
            src->spikeBitmap = both; src->bitmapStride = words;
            r->bitmapsStale = true;
            m.srcBitmap = both; m.bitmapStride = words;
            // the other populations' blocks, numbered from 0
            std::vector<NeuronGroupDev> rest;
            uint32_t block = 0;
            for(const auto &n : r->neuron) {
                if(&n == target) { continue; }
                rest.push_back(n);
                rest.back().startBlock = block;
                rest.back().numBlocks = (n.g.numNeurons + CONV_STEP_THREADS * r->neuronsPerLane - 1) / (CONV_STEP_THREADS * r->neuronsPerLane);
                block += rest.back().numBlocks;
            }
            r->convRestBlocks = block;
            m.restBlocks = block; m.restNeuronsPerLane = r->neuronsPerLane;
            HIP_TRY(hipMemcpy(r->dConvMfma, &m, sizeof(ConvMfmaDev), hipMemcpyHostToDevice));
            HIP_TRY(uploadPerBlock(rest, r->convRestBlocks, &r->dConvRest));
            HIP_TRY(hipMalloc(&r->dConvTarget, sizeof(NeuronGroupDev)));
            HIP_TRY(hipMemcpy(r->dConvTarget, target, sizeof(NeuronGroupDev), hipMemcpyHostToDevice));
            const size_t aggCount = 2 * (size_t)r->convMfmaBlocks * r->batch, restCount = 2 * (size_t)std::max(1u, r->convRestBlocks) * r->batch;
            HIP_TRY(hipMalloc(&r->dConvAgg, aggCount * sizeof(unsigned long long)));
            HIP_TRY(hipMemset(r->dConvAgg, 0, aggCount * sizeof(unsigned long long)));
            HIP_TRY(hipMalloc(&r->dConvRestAgg, restCount * sizeof(unsigned long long)));
            HIP_TRY(hipMemset(r->dConvRestAgg, 0, restCount * sizeof(unsigned long long)));
            for(void *q : {(void*)r->dConvRest, (void*)r->dConvTarget, (void*)r->dConvAgg, (void*)r->dConvRestAgg}) { if(q) { r->owned.push_back(q); } }
            r->convStepBytes = bytes;
            if(bytes > 48 * 1024) {
                HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void*>(convStepKernel), hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes));
            }
            r->convStep = true;
        }
    }
    HIP_TRY(uploadPerBlock(r->neuron, r->neuronBlocks, &r->dNeuron));
    HIP_TRY(uploadPerBlock(r->pre, r->preBlocks, &r->dPre));
    HIP_TRY(uploadPerBlock(r->post, r->postBlocks, &r->dPost));
    HIP_TRY(uploadPerBlock(r->dense, r->denseBlocks, &r->dDense));
    HIP_TRY(uploadPerBlock(r->proc, r->procBlocks, &r->dProc));
    const size_t aggCount = 2 * (size_t)r->neuronBlocks * r->batch;       // per-block counts, then per-group totals
    HIP_TRY(hipMalloc(&r->dAgg, aggCount * sizeof(unsigned long long)));
    HIP_TRY(hipMemset(r->dAgg, 0, aggCount * sizeof(unsigned long long)));
    if(!r->ordered) { const int rc = setupResident(r, numCU); if(rc) { return rc; } }
    if(const char *envSpin = getenv("GENNMI_SPIN_LIMIT")) {
        const uint32_t limit = (uint32_t)std::max(0ll, atoll(envSpin));
        HIP_TRY(hipMemcpyToSymbol(HIP_SYMBOL(c_spinLimit), &limit, sizeof(limit)));
    }
    else {
        const uint32_t limit = SPIN_LIMIT;
        HIP_TRY(hipMemcpyToSymbol(HIP_SYMBOL(c_spinLimit), &limit, sizeof(limit)));
    }
    HIP_TRY(hipDeviceSynchronize());
    r->finalised = true;
    return GENNMI_OK;
}

// Timing: events are taken from a pool and recorded on the runner's stream around each kernel; elapsed times are
// only read (after one synchronisation) when the pool is full or statistics are requested.
static int drainTimers(gennmi_runner *r)
{
    if(r->pending.empty()) { return GENNMI_OK; }
    HIP_TRY(hipStreamSynchronize(r->stream));
    for(const auto &p : r->pending) {
        float ms = 0;
        HIP_TRY(hipEventElapsedTime(&ms, p.a, p.b));
        const double sec = ms * 1e-3;
        if(p.kind == 0) { r->preTime += sec; r->preLaunches++; }
        else if(p.kind == 1) { r->postTime += sec; r->postLaunches++; }
        else if(p.kind == 2) { r->neuronTime += sec; r->neuronLaunches++; }
        else { r->stepTime += sec; r->stepLaunches++; }
    }
    r->pending.clear();
    r->eventNext = 0;
    return GENNMI_OK;
}

static int stamp(gennmi_runner *r, hipEvent_t *out)
{
    if(r->eventNext == r->eventPool.size()) {
        hipEvent_t e;
        HIP_TRY(hipEventCreate(&e));
        r->eventPool.push_back(e);
    }
    *out = r->eventPool[r->eventNext++];
    HIP_TRY(hipEventRecord(*out, r->stream));
    return GENNMI_OK;
}

// spike sources: bring the per-neuron copies of the next spike time up to date with arrays written since they were built
static int refreshSpikeSources(gennmi_runner *r)
{
    bool stale, bitmaps;
    {
        std::lock_guard<std::mutex> lock(g_runnersMutex);
        stale = r->sourcesStale;
        r->sourcesStale = false;
        bitmaps = r->bitmapsStale;
        r->bitmapsStale = false;
    }
    if(bitmaps) {
        // a spike queue was written from outside (or held spikes before its bitmap existed): the bitmap follows the queue
        for(const auto &n : r->neuron) {
            if(!n.spikeBitmap || n.g.numDelaySlots > 1) { continue; }
            const uint32_t words = (n.g.numNeurons + 31) / 32;
            // (of two copies, the one the coming step reads: the update after k completed steps writes copy (k + 1) & 1)
            uint32_t *bitmap = n.spikeBitmap + (r->epoch & 1) * n.bitmapStride;
            spikeBitmapFromQueueKernel<<<dim3((words + BLOCK - 1) / BLOCK, r->batch), dim3(BLOCK), 0, r->stream>>>(n.g.spkCnt, n.g.spk, bitmap, n.g.numNeurons, 1u);
            spikeBitmapFromQueueKernel<<<dim3((n.g.numNeurons + BLOCK - 1) / BLOCK, r->batch), dim3(BLOCK), 0, r->stream>>>(n.g.spkCnt, n.g.spk, bitmap, n.g.numNeurons, 0u);
            HIP_TRY(hipGetLastError());
        }
    }
    if(!stale) { return GENNMI_OK; }
    for(const auto &n : r->neuron) {
        if(n.g.model != GENNMI_NEURON_SPIKE_SOURCE_ARRAY) { continue; }
        const size_t count = (size_t)r->batch * n.g.numNeurons;
        nextSpikeTimeKernel<<<dim3((unsigned int)((count + BLOCK - 1) / BLOCK)), dim3(BLOCK), 0, r->stream>>>(n.g.startSpike, n.g.endSpike, n.g.spikeTimes,
                                                                                                              n.nextSpikeTime, count);
        HIP_TRY(hipGetLastError());
    }
    return GENNMI_OK;
}

static int launchSynapses(gennmi_runner *r, const StepArgs &a, bool timed)
{
    hipEvent_t e0 = nullptr, e1 = nullptr, e2 = nullptr;
    bool postInCombined = false;
    if(timed) {
        if(r->pending.size() >= 2048) { const int rc = drainTimers(r); if(rc) { return rc; } }
        const int rc = stamp(r, &e0); if(rc) { return rc; }
    }
    if(!r->pre.empty() || r->denseBlocks || r->procBlocks) {
        if(r->procBlocks) {
            presynapticProceduralKernel<<<dim3(r->procBlocks, r->batch), dim3(BLOCK), 0, r->stream>>>(r->dProc, r->dEvents);
        }
        if(r->ordered && !r->orderedGroups.empty()) {
            // the step's spikes as bitmaps, then one gather per projection, in push order: projections that share a
            // target add to it one after another, as the CPU backend's loop over its synapse groups does
            orderedClearKernel<<<dim3((unsigned int)((r->orderedBitmapWords + BLOCK - 1) / BLOCK)), dim3(BLOCK), 0, r->stream>>>(r->dOrderedBitmaps, r->orderedBitmapWords);
            orderedBitmapKernel<<<dim3(r->orderedSourceBlocks, r->batch), dim3(BLOCK), 0, r->stream>>>(r->dOrderedSources, a, r->dt);
            for(const auto &o : r->orderedGroups) {
                presynapticOrderedKernel<<<dim3((o.g.numTrgNeurons + (BLOCK / WAVE) - 1) / (BLOCK / WAVE), r->batch), dim3(BLOCK), 0, r->stream>>>(o, a, r->dt, r->dEvents);
            }
        }
        // (timed runs keep a launch per kernel, so that presynaptic and postsynaptic time stay apart as the reference reports them)
        const bool combined = r->combineSynapses && !timed;
        if(combined) {
            const uint32_t scatterBlocks = (r->preBlocks && r->scatterNeeded) ? r->preBlocks : 0u;
            const uint32_t postBlocks = r->combinePost ? r->postBlocks : 0u;
            postInCombined = (postBlocks != 0);
            synapseCombinedKernel<<<dim3(scatterBlocks + r->tileBlocks + postBlocks, r->batch), dim3(r->synapseThreads), r->combinedLdsBytes, r->stream>>>(
                r->dPre, scatterBlocks, r->dTile, r->tileBlocks, r->dPost, a, r->dt, r->dEvents);
        }
        else if(r->preBlocks && r->scatterNeeded && !(r->convMfmaBlocks && !timed)) {
            presynapticUpdateKernel<<<dim3(r->preBlocks, r->batch), dim3(r->synapseThreads), 0, r->stream>>>(r->dPre, a, r->dt, r->dEvents);
        }
        if(r->denseBlocks) {
            presynapticDenseKernel<<<dim3(r->denseBlocks, r->batch), dim3(BLOCK), 0, r->stream>>>(r->dDense, r->dEvents);
        }
        if(r->tileBlocks && !combined) {
            presynapticTileKernel<<<dim3(r->tileBlocks, r->batch), dim3(r->tileThreads), r->tileFloats * sizeof(float), r->stream>>>(r->dTile, a, r->dt, r->dEvents);
        }
        if(r->convMfmaBlocks) {
            // (the scatter blocks of the projection ride along unless the run is timed)
            const uint32_t scatterBlocks = (r->preBlocks && r->scatterNeeded && !timed) ? r->preBlocks : 0u;
            presynapticConvMfmaKernel<<<dim3((r->convMfmaBlocks + scatterBlocks) * r->batch), dim3(CONV_MFMA_THREADS), r->convMfmaBytes, r->stream>>>(
                r->dConvMfma, r->convMfmaBlocks * r->batch, r->dPre, a, r->dt, r->dEvents);
        }
        if(r->convTileBlocks) {
            presynapticConvTileKernel<<<dim3(r->convTileBlocks, r->batch), dim3(CONV_TILE_THREADS), r->convTileBytes, r->stream>>>(r->dConvTile, r->dEvents);
        }
        if(timed) { const int rc = stamp(r, &e1); if(rc) { return rc; } r->pending.push_back({e0, e1, 0}); }
    }
    if(!r->post.empty() && !postInCombined) {
        postsynapticUpdateKernel<<<dim3(r->postBlocks, r->batch), dim3(r->synapseThreads), r->postLdsBytes, r->stream>>>(r->dPost, a, r->dt);
        if(timed) { const int rc = stamp(r, &e2); if(rc) { return rc; } r->pending.push_back({e1 ? e1 : e0, e2, 1}); }
    }
    HIP_TRY(hipGetLastError());
    return GENNMI_OK;
}

static int launchNeurons(gennmi_runner *r, const StepArgs &a, bool timed);

static int launchFusedStep(gennmi_runner *r, const StepArgs &a)
{
    stepFusedKernel<<<dim3(r->neuronBlocks + r->preBlocks, r->batch), dim3(BLOCK), 0, r->stream>>>(
        r->dNeuron, r->neuronBlocks, r->dPre, a, r->dt, r->dAgg, r->dError, r->dEvents);
    HIP_TRY(hipGetLastError());
    return GENNMI_OK;
}

static int launchConvStep(gennmi_runner *r, const StepArgs &a)
{
    convStepKernel<<<dim3((r->convMfmaBlocks + r->convRestBlocks) * r->batch), dim3(CONV_STEP_THREADS), r->convStepBytes, r->stream>>>(
        r->dConvMfma, r->dConvTarget, r->dConvRest, r->batch, a, r->dt, r->dConvAgg, r->dConvRestAgg, r->dError, r->dEvents);
    HIP_TRY(hipGetLastError());
    return GENNMI_OK;
}

// one whole timestep: a single launch where the runner allows it, else synapse kernels then the neuron kernel
static int launchStep(gennmi_runner *r, const StepArgs &a)
{
    if(r->fusedStep) { return launchFusedStep(r, a); }
    if(r->convStep) { return launchConvStep(r, a); }
    const int rc = launchSynapses(r, a, false);
    return rc ? rc : launchNeurons(r, a, false);
}

static int launchNeurons(gennmi_runner *r, const StepArgs &a, bool timed)
{
    hipEvent_t e0 = nullptr, e1 = nullptr;
    if(timed) { const int rc = stamp(r, &e0); if(rc) { return rc; } }
    const dim3 neuronGrid(r->neuronBlocks, r->batch);
    if(r->neuronsPerLane == 2) { neuronBulkKernel<2><<<neuronGrid, dim3(BLOCK), 0, r->stream>>>(r->dNeuron, a, r->dt, r->dAgg, r->dError); }
    else if(r->neuronsPerLane == 4) { neuronBulkKernel<4><<<neuronGrid, dim3(BLOCK), 0, r->stream>>>(r->dNeuron, a, r->dt, r->dAgg, r->dError); }
    else if(r->neuronsPerLane == 8) { neuronBulkKernel<8><<<neuronGrid, dim3(BLOCK), 0, r->stream>>>(r->dNeuron, a, r->dt, r->dAgg, r->dError); }
    else { neuronUpdateKernel<<<dim3(r->neuronBlocks, r->batch), dim3(BLOCK), 0, r->stream>>>(r->dNeuron, a, r->dt, r->dAgg, r->dError); }
    if(timed) { const int rc = stamp(r, &e1); if(rc) { return rc; } r->pending.push_back({e0, e1, 2}); }
    HIP_TRY(hipGetLastError());
    return GENNMI_OK;
}

int gennmi_update_synapses(gennmi_runner *r, float t)
{
    if(!r || !r->finalised) { return fail(GENNMI_ESTATE, "update_synapses: runner not finalised"); }
    if(r->failed) { return fail(GENNMI_ESTATE, "update_synapses: an earlier queued step of this runner failed, the runner cannot continue"); }
    FLUSH_QUEUED();
    { const int rc = refreshTables(r); if(rc) { return rc; } }
    StepArgs a{};
    a.base = nullptr; a.epoch = r->epoch; a.t = t; a.recordingTimestep = 0;
    const int rc = launchSynapses(r, a, r->timing);
    if(rc) { return rc; }
    r->synapsesDone = true;
    return GENNMI_OK;
}

int gennmi_update_neurons(gennmi_runner *r, float t, uint32_t recordingTimestep)
{
    if(!r || !r->finalised) { return fail(GENNMI_ESTATE, "update_neurons: runner not finalised"); }
    if(r->failed) { return fail(GENNMI_ESTATE, "update_neurons: an earlier queued step of this runner failed, the runner cannot continue"); }
    FLUSH_QUEUED();
    { const int rc = refreshSpikeSources(r); if(rc) { return rc; } }
    StepArgs a{};
    a.base = nullptr; a.epoch = r->epoch; a.t = t; a.recordingTimestep = recordingTimestep;
    const int rc = launchNeurons(r, a, r->timing);
    if(rc) { return rc; }
    r->epoch++;
    r->synapsesDone = false;
    return GENNMI_OK;
}

int gennmi_step_time(gennmi_runner *r, unsigned long long timestep, unsigned long long numRecordingTimesteps)
{
    if(!r) { return fail(GENNMI_EINVAL, "step_time: null runner"); }
    // const float t = timestep * DT  (generateRunner.cc:283)
    const float t = (float)timestep * r->dt;
    const uint32_t recT = numRecordingTimesteps ? (uint32_t)(timestep % numRecordingTimesteps) : 0u;
    return gennmi_step(r, t, recT);
}

// one step, launched now
static int stepNow(gennmi_runner *r, float t, uint32_t recordingTimestep)
{
    if(r->fusedStep || r->convStep) {
        StepArgs a{};
        a.base = nullptr; a.epoch = r->epoch; a.t = t; a.recordingTimestep = recordingTimestep;
        hipEvent_t e0 = nullptr, e1 = nullptr;
        if(r->timing) {
            if(r->pending.size() >= 2048) { const int rc = drainTimers(r); if(rc) { return rc; } }
            const int rc = stamp(r, &e0); if(rc) { return rc; }
        }
        const int rc = r->fusedStep ? launchFusedStep(r, a) : launchConvStep(r, a);
        if(rc) { return rc; }
        if(r->timing) { const int rc2 = stamp(r, &e1); if(rc2) { return rc2; } r->pending.push_back({e0, e1, 3}); }
        r->epoch++;
        return GENNMI_OK;
    }
    const int rc = gennmi_update_synapses(r, t);
    if(rc) { return rc; }
    return gennmi_update_neurons(r, t, recordingTimestep);
}

// Executes the steps a runner has queued: runs of steps whose recording rows follow one another (or that all record into row
// 0: no recording, or a one-row buffer) go to the resident kernel in one launch, anything shorter than it accepts step by step.
static int flushRunnerSteps(gennmi_runner *r, const std::vector<gennmi_runner::QueuedStep> &steps);
// (The queue belongs to the thread that steps the runner: one host thread per runner.)
static int flushRunner(gennmi_runner *r)
{
    if(r->queued.empty()) { return GENNMI_OK; }
    std::vector<gennmi_runner::QueuedStep> steps;
    steps.swap(r->queued);
    g_queuedRunners--;
    const int rc = flushRunnerSteps(r, steps);
    // steps behind a failed one cannot be run later (the network's state is that of a step half done): say so from now on
    if(rc) { r->failed = true; }
    return rc;
}
static int flushRunnerSteps(gennmi_runner *r, const std::vector<gennmi_runner::QueuedStep> &steps)
{
    { const int rc = refreshSpikeSources(r); if(rc) { return rc; } }
    { const int rc = refreshTables(r); if(rc) { return rc; } }
    size_t first = 0;
    while(first < steps.size()) {
        size_t end = first + 1;
        const bool flat = (end < steps.size() && steps[first].recordingTimestep == 0 && steps[end].recordingTimestep == 0);
        while(end < steps.size() && steps[end].recordingTimestep == (flat ? 0u : steps[end - 1].recordingTimestep + 1u)) { end++; }
        const size_t count = end - first;
        if(r->resident && !r->timing && count >= 4) {
            // the kernel records step k of the launch into row (timestep + k) % numRecordingTimesteps
            const int rc = flat ? launchResident(r, 0, count, 1) : launchResident(r, steps[first].recordingTimestep, count, 1ull << 32);
            if(rc) { return rc; }
        }
        else {
            for(size_t k = first; k < end; k++) {
                const int rc = stepNow(r, steps[k].t, steps[k].recordingTimestep);
                if(rc) { return rc; }
            }
        }
        first = end;
    }
    return GENNMI_OK;
}

int gennmi_runner_set_step_queue(gennmi_runner *r, uint32_t maxSteps)
{
    if(!r) { return fail(GENNMI_EINVAL, "runner_set_step_queue: null runner"); }
    { const int rc = flushRunner(r); if(rc) { return rc; } }
    r->stepQueueLimit = maxSteps;
    return GENNMI_OK;
}

int gennmi_step(gennmi_runner *r, float t, uint32_t recordingTimestep)
{
    if(!r || !r->finalised) { return fail(GENNMI_ESTATE, "step: runner not finalised"); }
    if(r->failed) { return fail(GENNMI_ESTATE, "step: an earlier queued step of this runner failed, the runner cannot continue"); }
    if(r->stepQueueLimit && r->resident && !r->timing) {
        if(r->queued.empty()) { g_queuedRunners++; }
        r->queued.push_back({t, recordingTimestep});
        return (r->queued.size() >= r->stepQueueLimit) ? flushRunner(r) : GENNMI_OK;
    }
    FLUSH_QUEUED();
    { const int rc = refreshSpikeSources(r); if(rc) { return rc; } }
    { const int rc = refreshTables(r); if(rc) { return rc; } }
    return stepNow(r, t, recordingTimestep);
}

int gennmi_run_steps(gennmi_runner *r, unsigned long long timestep, unsigned long long numSteps, unsigned long long numRecordingTimesteps)
{
    if(!r || !r->finalised) { return fail(GENNMI_ESTATE, "run_steps: runner not finalised"); }
    if(r->failed) { return fail(GENNMI_ESTATE, "run_steps: an earlier queued step of this runner failed, the runner cannot continue"); }
    FLUSH_QUEUED();
    { const int rc = refreshSpikeSources(r); if(rc) { return rc; } }
    { const int rc = refreshTables(r); if(rc) { return rc; } }
    constexpr unsigned long long CHUNK = 100;
    // (the resident plan takes time, epoch and recording length as kernel arguments: no step state on the device to refresh,
    // and so no copy and no wait for it ahead of the launch — 20 us of a call that launches 20 steps, and, between two
    // events recorded around the call, 20 us that are not the kernel's)
    if(r->resident && !r->timing && numSteps >= 4) { return launchResident(r, timestep, numSteps, numRecordingTimesteps); }
    const StepState hs{timestep, r->epoch, numRecordingTimesteps};
    HIP_TRY(hipMemcpyAsync(r->dState, &hs, sizeof(hs), hipMemcpyHostToDevice, r->stream));
    HIP_TRY(hipStreamSynchronize(r->stream));   // hs lives on this stack frame
    unsigned long long done = 0;
    if(r->timing) {
        // individually launched steps with HIP events around every kernel; nothing waits until the statistics
        // are read, so the device stays busy and the clocks stay up
        for(; done < numSteps; done++) {
            const int rc = gennmi_step_time(r, timestep + done, numRecordingTimesteps);
            if(rc) { return rc; }
        }
        return GENNMI_OK;
    }
    while(numSteps - done >= CHUNK) {
        if(!r->graphExec) {
            hipGraph_t graph;
            HIP_TRY(hipStreamBeginCapture(r->stream, hipStreamCaptureModeThreadLocal));
            int rc = GENNMI_OK;
            for(unsigned long long k = 0; k < CHUNK && rc == GENNMI_OK; k++) {
                StepArgs a{};
                a.base = r->dState; a.k = k;
                rc = launchStep(r, a);
            }
            advanceStepKernel<<<dim3(1), dim3(64), 0, r->stream>>>(r->dState, CHUNK);
            const hipError_t ce = hipStreamEndCapture(r->stream, &graph);
            if(rc) { return rc; }
            if(ce != hipSuccess) { return fail(GENNMI_EHIP, std::string("hipStreamEndCapture: ") + hipGetErrorString(ce)); }
            HIP_TRY(hipGraphInstantiate(&r->graphExec, graph, nullptr, nullptr, 0));
            HIP_TRY(hipGraphDestroy(graph));
            r->graphSteps = CHUNK;
        }
        HIP_TRY(hipGraphLaunch(r->graphExec, r->stream));
        done += CHUNK;
        r->epoch += CHUNK;
    }
    for(; done < numSteps; done++) {
        StepArgs a{};
        a.base = r->dState; a.k = 0;
        const int rc = launchStep(r, a);
        if(rc) { return rc; }
        advanceStepKernel<<<dim3(1), dim3(64), 0, r->stream>>>(r->dState, 1);
        r->epoch++;
    }
    HIP_TRY(hipGetLastError());
    return GENNMI_OK;
}

int gennmi_runner_synchronize(gennmi_runner *r)
{
    if(!r) { return fail(GENNMI_EINVAL, "runner_synchronize: null runner"); }
    FLUSH_QUEUED();
    // (the flag is host memory the kernels write: nothing to copy, it is read below once the stream has drained)
    // (short waits are polled: a blocking wait wakes up some tens of microseconds after the work has ended; GENNMI_POLL_US=0 blocks at once)
    static const long pollMicroseconds = [] { const char *e = getenv("GENNMI_POLL_US"); return e ? atol(e) : 500l; }();
    if(pollMicroseconds > 0) {
        const auto begin = std::chrono::steady_clock::now();
        hipError_t state = hipStreamQuery(r->stream);
        while(state == hipErrorNotReady && std::chrono::steady_clock::now() - begin < std::chrono::microseconds(pollMicroseconds)) { state = hipStreamQuery(r->stream); }
        (void)hipGetLastError();    // "not ready" is an answer, not a failure to keep
        if(state != hipSuccess && state != hipErrorNotReady) { HIP_TRY(state); }
    }
    HIP_TRY(hipStreamSynchronize(r->stream));
    const uint32_t err = *r->hError;
    if(err) { return fail(GENNMI_EDEVICE, "a kernel's bounded wait for other work-groups expired (spike offsets or spike exchange); state is undefined"); }
    return GENNMI_OK;
}

int gennmi_runner_set_timing(gennmi_runner *r, int enabled)
{
    if(!r) { return fail(GENNMI_EINVAL, "runner_set_timing: null runner"); }
    FLUSH_QUEUED();
    if(!enabled) { const int rc = drainTimers(r); if(rc) { return rc; } }
    r->timing = (enabled != 0);
    return GENNMI_OK;
}

int gennmi_runner_get_times(gennmi_runner *r, double *neuronUpdateTime, double *presynapticUpdateTime, double *postsynapticUpdateTime)
{
    if(!r) { return fail(GENNMI_EINVAL, "runner_get_times: null runner"); }
    FLUSH_QUEUED();
    { const int rc = drainTimers(r); if(rc) { return rc; } }
    // a single-launch step is one kernel that holds the neuron update and, in blocks of its own, the presynaptic update of the
    // previous step's spikes: its whole duration counts as neuron update time (the reference has no such kernel)
    if(neuronUpdateTime) { *neuronUpdateTime = r->neuronTime + r->stepTime; }
    if(presynapticUpdateTime) { *presynapticUpdateTime = r->preTime; }
    if(postsynapticUpdateTime) { *postsynapticUpdateTime = r->postTime; }
    return GENNMI_OK;
}

int gennmi_runner_kernel_stats(gennmi_runner *r, double stats[8])
{
    if(!r || !stats) { return fail(GENNMI_EINVAL, "runner_kernel_stats: null argument"); }
    FLUSH_QUEUED();
    { const int rc = drainTimers(r); if(rc) { return rc; } }
    stats[0] = (double)r->preLaunches; stats[1] = r->preTime;
    stats[2] = (double)r->neuronLaunches; stats[3] = r->neuronTime;
    stats[4] = (double)r->postLaunches; stats[5] = r->postTime;
    stats[6] = (double)r->stepLaunches; stats[7] = r->stepTime;
    return GENNMI_OK;
}

int gennmi_runner_stream_mark(gennmi_runner *r, int which)
{
    if(!r || which < 0 || which > 1) { return fail(GENNMI_EINVAL, "runner_stream_mark: bad arguments"); }
    FLUSH_QUEUED();
    if(!r->marks[which]) { HIP_TRY(hipEventCreate(&r->marks[which])); }
    HIP_TRY(hipEventRecord(r->marks[which], r->stream));
    return GENNMI_OK;
}

int gennmi_runner_stream_elapsed(gennmi_runner *r, double *seconds)
{
    if(!r || !seconds || !r->marks[0] || !r->marks[1]) { return fail(GENNMI_EINVAL, "runner_stream_elapsed: both marks must have been recorded"); }
    HIP_TRY(hipEventSynchronize(r->marks[1]));
    float ms = 0;
    HIP_TRY(hipEventElapsedTime(&ms, r->marks[0], r->marks[1]));
    *seconds = ms * 1e-3;
    return GENNMI_OK;
}

int gennmi_runner_get_info(gennmi_runner *r, uint32_t info[4])
{
    if(!r || !info) { return fail(GENNMI_EINVAL, "runner_get_info: null argument"); }
    if(!r->finalised) { return fail(GENNMI_ESTATE, "runner_get_info: runner not finalised"); }
    info[0] = (r->fusedStep ? 1u : 0u) | (r->resident ? 2u : 0u) | (r->neuronsPerLane > 1 ? 4u : 0u) | (r->ordered ? 8u : 0u)
              | (r->combineSynapses ? 16u : 0u) | ((r->combineSynapses && r->combinePost) ? 32u : 0u) | (r->convMfmaBlocks ? 64u : 0u) | (r->convStep ? 128u : 0u); info[1] = r->neuronBlocks; info[2] = r->preBlocks; info[3] = r->postBlocks;
    return GENNMI_OK;
}

int gennmi_runner_event_count(gennmi_runner *r, unsigned long long *events)
{
    if(!r || !events) { return fail(GENNMI_EINVAL, "runner_event_count: null argument"); }
    FLUSH_QUEUED();
    HIP_TRY(hipStreamSynchronize(r->stream));
    // (partial counts a cache line apart: see addEvents)
    unsigned long long slots[EVENT_SLOTS * EVENT_SLOT_STRIDE];
    HIP_TRY(hipMemcpy(slots, r->dEvents, sizeof(slots), hipMemcpyDeviceToHost));
    unsigned long long total = 0;
    for(uint32_t k = 0; k < EVENT_SLOTS; k++) { total += slots[k * EVENT_SLOT_STRIDE]; }
    *events = total;
    return GENNMI_OK;
}

int gennmi_max_col_length(uint32_t numSrc, uint32_t numTrg, uint32_t rowStride, const uint32_t *rowLength, const uint32_t *ind, uint32_t *maxColLength)
{
    if(!rowLength || !ind || !maxColLength || rowStride == 0) { return fail(GENNMI_EINVAL, "max_col_length: bad arguments"); }
    FLUSH_QUEUED();
    uint32_t *dCount = nullptr;
    HIP_TRY(hipMalloc(&dCount, (size_t)numTrg * sizeof(uint32_t)));
    HIP_TRY(hipMemset(dCount, 0, (size_t)numTrg * sizeof(uint32_t)));
    const size_t total = (size_t)numSrc * rowStride;
    remapCountKernel<<<dim3((unsigned int)((total + BLOCK - 1) / BLOCK)), dim3(BLOCK), 0, 0>>>(numSrc, rowStride, rowLength, ind, 0, dCount, nullptr, nullptr);
    HIP_TRY(hipGetLastError());
    std::vector<uint32_t> h(numTrg);
    HIP_TRY(hipMemcpy(h.data(), dCount, (size_t)numTrg * sizeof(uint32_t), hipMemcpyDeviceToHost));
    HIP_TRY(hipFree(dCount));
    uint32_t m = 0;
    for(uint32_t v : h) { m = std::max(m, v); }
    *maxColLength = m;
    return GENNMI_OK;
}

// ---- the one entry point that allocates nothing: gennmi_max_col_length with its per-column counters in a file-scope
// device array instead of a hipMalloc'd one.  Every device holds its own copy of the array at its own address; the
// address is looked up once per device and that pointer — never the array's name, which in host code is only a
// handle — is what the kernels receive.
}   // extern "C"

namespace
{
constexpr uint32_t STATIC_COUNTER_MAX = GENNMI_STATIC_MAX_TARGETS;       // 2^20 counters = 4 MiB per device
static __device__ __align__(256) uint32_t scratch[STATIC_COUNTER_MAX];
constexpr int STATIC_MAX_DEVICES = 64;
std::mutex g_scratchMutex;
uint32_t *g_scratchPtr[STATIC_MAX_DEVICES] = {};

// clears the counters a call will use and its result word
__global__ void staticClearKernel(uint32_t *counters, uint32_t count, uint32_t *result)
{
    const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
    if(i < count) { counters[i] = 0u; }
    if(i == 0) { *result = 0u; }
}

__global__ __launch_bounds__(BLOCK)
void staticMaxKernel(const uint32_t *counters, uint32_t count, uint32_t *result)
{
    const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
    uint32_t v = (i < count) ? counters[i] : 0u;
    for(int off = WAVE / 2; off > 0; off >>= 1) { v = max(v, (uint32_t)__shfl_down(v, off, WAVE)); }
    if((threadIdx.x & (WAVE - 1)) == 0 && v) { atomicMax(result, v); }
}

// address of the current device's copy of `scratch` (looked up on first use, once per device)
int staticScratch(uint32_t **ptr)
{
    int device = 0;
    HIP_TRY(hipGetDevice(&device));
    if(device < 0 || device >= STATIC_MAX_DEVICES) { return fail(GENNMI_EUNSUPPORTED, "static scratch: device index out of range"); }
    std::lock_guard<std::mutex> lock(g_scratchMutex);
    if(!g_scratchPtr[device]) {
        uint32_t *p = nullptr;
        HIP_TRY(hipGetSymbolAddress((void**)&p, HIP_SYMBOL(scratch)));
        if(!p) { return fail(GENNMI_EHIP, "static scratch: hipGetSymbolAddress returned a null address"); }
        g_scratchPtr[device] = p;
    }
    *ptr = g_scratchPtr[device];
    return GENNMI_OK;
}
}   // namespace

int gennmi_detail::prepareStaticScratch()
{
    uint32_t *unused = nullptr;
    return staticScratch(&unused);
}

extern "C" {

int gennmi_max_col_length_static(uint32_t numSrc, uint32_t numTrg, uint32_t rowStride, const uint32_t *rowLength, const uint32_t *ind,
                                 uint32_t *maxColLengthDev)
{
    if(!rowLength || !ind || !maxColLengthDev || rowStride == 0 || numSrc == 0 || numTrg == 0) { return fail(GENNMI_EINVAL, "max_col_length_static: bad arguments"); }
    if(numTrg > STATIC_COUNTER_MAX) {
        return fail(GENNMI_EINVAL, "max_col_length_static: " + std::to_string(numTrg) + " postsynaptic neurons exceed the static counter array ("
                                   + std::to_string(STATIC_COUNTER_MAX) + "); use gennmi_max_col_length");
    }
    const size_t total = (size_t)numSrc * rowStride;
    if((total + BLOCK - 1) / BLOCK > 0x7FFFFFFFull) { return fail(GENNMI_EINVAL, "max_col_length_static: matrix too large for one launch"); }
    uint32_t *counters = nullptr;
    { const int rc = staticScratch(&counters); if(rc) { return rc; } }
    // the array keeps the last call's counts: clear what this call uses
    staticClearKernel<<<dim3((numTrg + BLOCK - 1) / BLOCK), dim3(BLOCK), 0, 0>>>(counters, numTrg, maxColLengthDev);
    remapCountKernel<<<dim3((unsigned int)((total + BLOCK - 1) / BLOCK)), dim3(BLOCK), 0, 0>>>(numSrc, rowStride, rowLength, ind, 0, counters, nullptr, nullptr);
    staticMaxKernel<<<dim3((numTrg + BLOCK - 1) / BLOCK), dim3(BLOCK), 0, 0>>>(counters, numTrg, maxColLengthDev);
    HIP_TRY(hipGetLastError());
    return GENNMI_OK;
}

int gennmi_build_remap(uint32_t numSrc, uint32_t numTrg, uint32_t rowStride, uint32_t colStride,
                       const uint32_t *rowLength, const uint32_t *ind, uint32_t *colLength, uint32_t *remap)
{
    if(!rowLength || !ind || !colLength || !remap || rowStride == 0 || colStride == 0) { return fail(GENNMI_EINVAL, "build_remap: bad arguments"); }
    FLUSH_QUEUED();
    uint32_t *dOverflow = nullptr;
    HIP_TRY(hipMalloc(&dOverflow, sizeof(uint32_t)));
    HIP_TRY(hipMemset(dOverflow, 0, sizeof(uint32_t)));
    HIP_TRY(hipMemset(colLength, 0, (size_t)numTrg * sizeof(uint32_t)));
    const size_t total = (size_t)numSrc * rowStride;
    remapCountKernel<<<dim3((unsigned int)((total + BLOCK - 1) / BLOCK)), dim3(BLOCK), 0, 0>>>(numSrc, rowStride, rowLength, ind, colStride, colLength, remap, dOverflow);
    HIP_TRY(hipGetLastError());
    uint32_t overflow = 0;
    HIP_TRY(hipMemcpy(&overflow, dOverflow, sizeof(uint32_t), hipMemcpyDeviceToHost));
    HIP_TRY(hipFree(dOverflow));
    if(overflow) { return fail(GENNMI_EINVAL, "build_remap: a column holds " + std::to_string(overflow) + " synapses, more than colStride"); }
    const size_t lds = (size_t)pow2Ceil(std::min(colStride, REMAP_SORT_MAX)) * sizeof(uint32_t);
    if(lds > 48 * 1024) {
        HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void*>(remapSortKernel), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    }
    remapSortKernel<<<dim3(numTrg), dim3(BLOCK), lds, 0>>>(colStride, colLength, remap);
    // columns beyond what the LDS holds, in place in global memory
    if(colStride > REMAP_SORT_MAX) { remapSortLongKernel<<<dim3(numTrg), dim3(BLOCK), 0, 0>>>(colStride, colLength, remap); }
    HIP_TRY(hipGetLastError());
    HIP_TRY(hipDeviceSynchronize());
    return GENNMI_OK;
}

}   // extern "C"

// generated code objects behind the C ABI: gennmi_program_*
#include "genn_mi355x_program.h"
