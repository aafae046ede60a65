// MI355X (gfx950) device layer for GeNN's per-timestep hot path: kernels + C ABI.
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
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <type_traits>
#include <map>
#include <mutex>
#include <vector>

#include "genn_mi355x.h"
#include "genn_mi355x_rows.h"

namespace
{
constexpr int BLOCK = 256;                  // 4 wave64 per work-group
constexpr int WAVE = 64;
constexpr int CONV_TILE_SPIKES = 2048;      // spikes staged in LDS at a time by the Conv2D tile kernel
constexpr int CONV_TILE_THREADS = 512;      // work-group size of the Conv2D tile kernel (8 wave64 share one LDS tile)
constexpr uint32_t SPIN_LIMIT = 1u << 22;   // default bound of every wait for another work-group (polls)
constexpr uint32_t REMAP_SORT_MAX = 16384;  // longest column the LDS sort handles (64 KiB)

thread_local std::string g_lastError;

int fail(int code, const std::string &msg)
{
    g_lastError = msg;
    return code;
}

#define HIP_TRY(expr)                                                                              \
    do {                                                                                           \
        hipError_t e_ = (expr);                                                                    \
        if(e_ != hipSuccess) {                                                                     \
            return fail(GENNMI_EHIP, std::string(#expr) + ": " + hipGetErrorString(e_));           \
        }                                                                                          \
    } while(0)

// Polls a work-group spends waiting for another one before it raises the error flag and leaves.  Set from
// GENNMI_SPIN_LIMIT when a runner is finalised; tests of the failure path set it to 0 so that the first missed poll expires.
__constant__ uint32_t c_spinLimit = SPIN_LIMIT;

// ------------------------------------------------------------------------------------------------
// device-side tables
// ------------------------------------------------------------------------------------------------
struct StepState             // device-resident; lets a captured graph be replayed unchanged
{
    unsigned long long timestep;
    unsigned long long epoch;           // number of completed steps since runner creation
    unsigned long long numRecordingTimesteps;
};

struct StepArgs              // per-launch; either direct values or offsets from *base
{
    const StepState *base;
    unsigned long long k;               // offset added to base->timestep / base->epoch
    unsigned long long epoch;           // direct
    float t;                            // direct
    uint32_t recordingTimestep;         // direct
};

struct Resolved { float t; uint32_t recT; unsigned long long epoch; };

// step counter modulo a 32-bit period: 64-bit division is a long software routine on this part, and the
// counter fits 32 bits for the first 4e9 steps
__device__ __forceinline__ uint32_t modStep(unsigned long long x, uint32_t d)
{
    return (x >> 32) ? (uint32_t)(x % d) : ((uint32_t)x % d);
}

__device__ __forceinline__ Resolved resolve(const StepArgs &a, float dt)
{
    Resolved r;
    if(a.base) {
        const unsigned long long ts = a.base->timestep + a.k;
        // const float t = timestep * DT  (generateRunner.cc:283)
        r.t = (float)ts * dt;
        const unsigned long long nr = a.base->numRecordingTimesteps;
        r.recT = nr ? (((ts | nr) >> 32) ? (uint32_t)(ts % nr) : ((uint32_t)ts % (uint32_t)nr)) : 0u;
        r.epoch = a.base->epoch + a.k;
    }
    else {
        r.t = a.t; r.recT = a.recordingTimestep; r.epoch = a.epoch;
    }
    return r;
}

// Synapses whose dendritic delay is a multiple of the ring depth land in the slot the target reads in
// the very step that delivers them.  When a runner handles them in the neuron update (see
// gennmi_runner_finalise), each population carries one of these per outgoing delayed projection:
// the positions of such synapses within every row.
struct ZeroDelayEntry
{
    float *ringElem;                    // &denDelay[ipost] of the target ring (slot 0, batch 0)
    const float *weight;                // &g[idSyn]: read at delivery time, so pushed weights are honoured
    uint32_t numTrgNeurons, maxDenDelay;
};

struct NeuronGroupDev
{
    gennmi_neuron_update_group_t g;
    uint32_t startBlock, numBlocks;
    const uint32_t *zeroStart;          // [N+1] CSR offsets into zeroEntries (all outgoing projections merged), or NULL
    const ZeroDelayEntry *zeroEntries;
    uint32_t *shadowSpk;                // [2][batch*N] engine-private double-buffered copy of the spike queue, or NULL
    uint32_t *shadowCnt;                // [2][batch]
    uint32_t *spikeBitmap;              // [ceil(N/32)] engine-private bitmap of this step's spikes (populations with learnPost), or NULL
    unsigned long long *aggEvent;       // look-back area of the spike-like event queues (groups with events), or NULL
    float *nextSpikeTime;               // spike sources: engine-private copy of spikeTimes[startSpike] per neuron (+inf: none left)
    size_t spikeTimesBytes;             // spike sources: bytes from spikeTimes to the end of its allocation (host bookkeeping)
};

struct PreGroupDev
{
    gennmi_presynaptic_update_group_t g;
    uint32_t startBlock, numBlocks;
    uint32_t lanesPerSpike;             // power of two, 1..64
    uint32_t vec4;                      // rows are 16-byte aligned and padded: dwordx4 loads
    int32_t convBH, convBW;
    uint32_t skipZeroDelay;             // synapses with d % D == 0 are delivered by the neuron update instead
    uint32_t tileThreshold;             // != 0: leave the step to the tile kernel when numSpikes*workPerSpike reaches it
    uint32_t workPerSpike, pad2_;       // rowStride (SPARSE) or kh*kw*oc (Toeplitz)
    const uint32_t *shadowSpk;          // the source population's shadow queue (read instead of srcSpk when set)
    const uint32_t *shadowCnt;
};

// Dense-activity path of a static SPARSE projection without delay: one block accumulates the events that
// fall into one tile of postsynaptic neurons in LDS and flushes the tile with lane-consecutive atomics.
struct TileGroupDev
{
    gennmi_presynaptic_update_group_t g;
    const uint16_t *tileOff;            // [numSrc*(numTiles+1)] first position of every row whose target is >= tile*tileSize
    uint32_t numTiles, tileSize;
    uint32_t tile, split, numSplits;    // this block: which tile, which share of the spikes
    uint32_t lanes;                     // lanes per (spike, tile) segment, power of two
    uint32_t threshold, pad_;
};

// Dense-activity path of a Toeplitz Conv2D projection: a block owns rowsPerTile output rows (all columns and
// channels) in LDS next to a copy of the kernel weights.
struct ConvTileDev
{
    gennmi_presynaptic_update_group_t g;
    int32_t convBH, convBW;
    uint32_t rowsPerTile, tileRow0;
    uint32_t threshold, pad_;
};

struct PostGroupDev
{
    gennmi_postsynaptic_update_group_t g;
    uint32_t startBlock, numBlocks;
    uint32_t lanesPerSpike;
    uint32_t denseThreshold;            // != 0: steps with at least this many postsynaptic spikes walk the rows instead
    const uint32_t *spikeBitmap;        // [ceil(numTrg/32)] this step's postsynaptic spikes, written by the neuron update
};

// Block -> group: groups occupy consecutive block ranges (the reference pads thread ranges to block
// multiples for the same reason, backendSIMT.h:244-323).  Every block has its own copy of its group's
// descriptor in a table indexed by blockIdx.x.

// Pointers reach the kernels through descriptor tables, so the compiler cannot know their address
// space; these casts let it emit global_load / global_atomic instead of flat instructions.
#define GLOBAL_AS __attribute__((address_space(1)))
template<typename T>
__device__ __forceinline__ GLOBAL_AS T *asGlobal(T *p) { return (GLOBAL_AS T*)p; }
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef uint8_t u8x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4u __attribute__((ext_vector_type(4), aligned(4)));     // dword-aligned only: segments start anywhere in a row
typedef float f32x4u __attribute__((ext_vector_type(4), aligned(4)));

__device__ __forceinline__ void atomicAddF32(GLOBAL_AS float *addr, float v)
{
    // gfx950 has a native global_atomic_add_f32; the old value is not needed
    __builtin_amdgcn_global_atomic_fadd_f32(addr, v);
}

// ------------------------------------------------------------------------------------------------
// Presynaptic update.  The unit of work is (spike, chunk of its row): a sub-group of
// `lanesPerSpike` lanes handles `span` consecutive synapses of one row, so a long row is spread
// over many wavefronts instead of being walked serially, and every load of ind / g / d is one
// contiguous segment (dwordx4 per lane when rows are padded to 4 entries and 16-byte aligned).
// lanesPerSpike = 64 is the "post span" mapping (lanes span the row); small values are the
// "pre span" mapping (few lanes per spike, many spikes per wavefront).  Work items are dealt
// round-robin to the sub-groups of the synapse group's blocks, so the launch geometry is fixed
// while the spike count lives on the device.
// ------------------------------------------------------------------------------------------------
__device__ __forceinline__ void presynapticBody(const PreGroupDev &G, uint32_t blockInKernel, const Resolved &st, float dt,
                                                unsigned long long *eventCounter)
{
    const gennmi_presynaptic_update_group_t &g = G.g;
    const uint32_t batch = blockIdx.y;
    const uint32_t W = G.lanesPerSpike;
    const uint32_t localBlock = blockInKernel - G.startBlock;
    const uint32_t lis = threadIdx.x & (W - 1);
    const uint32_t subGroup = (localBlock * BLOCK + threadIdx.x) / W;
    const uint32_t numSubGroups = (G.numBlocks * BLOCK) / W;
    // spikes of the previous step: the population's own queue, or (when this launch may run next to the
    // neuron update that refills that queue) the shadow copy written one step ago
    const uint32_t parity = (uint32_t)((st.epoch + 1) & 1);
    // axonal delay: the source's queue is a ring of slots; this projection reads the slot written axonalDelaySteps + 1
    // updates ago, (spkQuePtr + slots - delay) % slots with spkQuePtr = epoch % slots (backendBase.cc:207-216)
    const uint32_t slots = max(1u, g.numSrcDelaySlots);
    const uint32_t readSlot = (slots > 1) ? modStep(st.epoch + slots - g.axonalDelaySteps, slots) : 0u;
    GLOBAL_AS const uint32_t *cntPtr = G.shadowSpk ? asGlobal(G.shadowCnt) + (size_t)parity * gridDim.y + batch
                                                   : asGlobal(g.srcSpkCnt) + ((size_t)batch * slots + readSlot);
    GLOBAL_AS const uint32_t *spk = G.shadowSpk ? asGlobal(G.shadowSpk) + ((size_t)parity * gridDim.y + batch) * g.numSrcNeurons
                                                : asGlobal(g.srcSpk) + ((size_t)batch * slots + readSlot) * g.numSrcNeurons;
    // the first spike id this sub-group would handle is fetched together with the count, not after it (the
    // queue always holds numSrcNeurons entries, so any index below that is readable)
    const uint32_t sparseSpan = W * (G.vec4 ? 4u : 1u);
    const uint32_t sparseChunksPerRow = (g.rowStride + sparseSpan - 1) / sparseSpan;
    const uint32_t firstSpike = (g.matrix == GENNMI_MATRIX_SPARSE) ? spk[min(subGroup / max(sparseChunksPerRow, 1u), g.numSrcNeurons - 1)] : 0u;
    const uint32_t numSpikes = cntPtr[0];
    if(G.tileThreshold && (unsigned long long)numSpikes * G.workPerSpike >= G.tileThreshold) { return; }
    GLOBAL_AS float *outPost = asGlobal(g.outPost) + (size_t)batch * g.numTrgNeurons;
    unsigned long long events = 0;

    if(g.matrix == GENNMI_MATRIX_TOEPLITZ_CONV2D) {
        // initToeplitzConnectivitySnippet.h:116-137; lanes span the kh*kw*oc diagonals, so
        // consecutive lanes hit consecutive output channels (consecutive outPost addresses)
        const int kh = g.conv[0], kw = g.conv[1], iw = g.conv[3], ic = g.conv[4];
        const int oh = g.conv[5], ow = g.conv[6], oc = g.conv[7];
        const uint32_t numDiag = (uint32_t)(kh * kw * oc);
        const uint32_t chunksPerRow = (numDiag + W - 1) / W;
        GLOBAL_AS const float *kernel = asGlobal(g.g);
        // item = subGroup + k*numSubGroups, split into (spike, chunk) incrementally: no division in the loop
        const uint32_t stepSpike = numSubGroups / chunksPerRow, stepChunk = numSubGroups % chunksPerRow;
        uint32_t chunk = subGroup % chunksPerRow;
        for(unsigned long long s = subGroup / chunksPerRow; s < numSpikes; ) {
            const uint32_t j = chunk * W + lis;
            const uint32_t ipre = spk[s];
            s += stepSpike; chunk += stepChunk;
            if(chunk >= chunksPerRow) { chunk -= chunksPerRow; s++; }
            if(j < numDiag) {
                const int preRow = (int)(ipre / ic) / iw;
                const int preCol = (int)(ipre / ic) % iw;
                const int preChan = (int)(ipre % ic);
                const int kernRow = (int)(j / oc) / kw;
                const int kernCol = (int)(j / oc) % kw;
                const int kernOutChan = (int)(j % oc);
                const int postRow = preRow + kernRow - G.convBH;
                const int postCol = preCol + kernCol - G.convBW;
                if(postRow >= 0 && postCol >= 0 && postRow < oh && postCol < ow) {
                    const int postInd = (postRow * ow * oc) + (postCol * oc) + kernOutChan;
                    const int kernelInd = ((kh - kernRow - 1) * kw * ic * oc) + ((kw - kernCol - 1) * ic * oc) + (preChan * oc) + kernOutChan;
                    atomicAddF32(&outPost[postInd], kernel[kernelInd]);
                    events++;
                }
            }
        }
    }
    else {
        const uint32_t D = g.maxDenDelay;
        // *denDelayPtr = (*denDelayPtr + 1) % D happens at the start of updateSynapses
        // (synapseUpdateGroupMerged.cc:480-483); st.epoch counts completed steps, so the pointer
        // in force during this step is (epoch + 1) % D.
        const uint32_t denPtr = D ? modStep(st.epoch + 1, D) : 0;
        GLOBAL_AS float *denDelay = D ? asGlobal(g.denDelay) + (size_t)batch * D * g.numTrgNeurons : nullptr;
        GLOBAL_AS const uint32_t *rowLength = asGlobal(g.rowLength);
        GLOBAL_AS const uint32_t *ind = asGlobal(g.ind);
        GLOBAL_AS float *weight = asGlobal(g.g);
        GLOBAL_AS const uint8_t *delay = asGlobal(g.d);
        const uint32_t numTrg = g.numTrgNeurons;
        const uint32_t perLane = G.vec4 ? 4u : 1u;
        const uint32_t span = W * perLane;
        const uint32_t chunksPerRow = (g.rowStride + span - 1) / span;
        // Loads are issued ahead of the values that decide whether they are needed, so that the
        // dependent chain per item is spike id -> {rowLength, row chunk} -> atomics: the spike id of
        // the NEXT item is fetched while the current one is processed (spk always holds
        // numSrcNeurons entries, so any index below that is readable), and the row chunk is read
        // together with rowLength (rows are padded to rowStride, so any j < rowStride is readable).
        const uint32_t lastSrc = g.numSrcNeurons - 1;
        uint32_t idPreNext = firstSpike;
        // item = subGroup + k*numSubGroups, split into (spike, chunk) incrementally: no division in the loop
        const uint32_t stepSpike = numSubGroups / chunksPerRow, stepChunk = numSubGroups % chunksPerRow;
        uint32_t chunkNext = subGroup % chunksPerRow;
        for(unsigned long long sNext = subGroup / chunksPerRow; sNext < numSpikes; ) {
            const uint32_t chunk = chunkNext;
            const uint32_t idPre = idPreNext;
            sNext += stepSpike; chunkNext += stepChunk;
            if(chunkNext >= chunksPerRow) { chunkNext -= chunksPerRow; sNext++; }
            idPreNext = spk[(uint32_t)min(sNext, (unsigned long long)lastSrc)];
            const size_t rowBase = (size_t)idPre * g.rowStride;
            const uint32_t j = chunk * span + lis * perLane;
            const bool inRow = (j < g.rowStride);
            const uint32_t npost = rowLength[idPre];
            if(g.wum == GENNMI_WUM_STATIC_PULSE) {
                if(G.vec4) {
                    u32x4 ip = {0, 0, 0, 0}; f32x4 w = {0, 0, 0, 0};
                    if(inRow) {
                        ip = *reinterpret_cast<GLOBAL_AS const u32x4*>(ind + rowBase + j);
                        w = *reinterpret_cast<GLOBAL_AS const f32x4*>(weight + rowBase + j);
                    }
                    if(j < npost) { atomicAddF32(&outPost[ip.x], w.x); }
                    if(j + 1 < npost) { atomicAddF32(&outPost[ip.y], w.y); }
                    if(j + 2 < npost) { atomicAddF32(&outPost[ip.z], w.z); }
                    if(j + 3 < npost) { atomicAddF32(&outPost[ip.w], w.w); }
                }
                else {
                    uint32_t ip = 0; float w = 0;
                    if(inRow) { ip = ind[rowBase + j]; w = weight[rowBase + j]; }
                    if(j < npost) { atomicAddF32(&outPost[ip], w); }
                }
            }
            else if(g.wum == GENNMI_WUM_STATIC_PULSE_DENDRITIC_DELAY) {
                // addToPostDelay(g, d): denDelay[((ptr + d) % D) * numPost + idPost] += g  (synapseUpdateGroupMerged.cc:245-251)
                if(G.vec4) {
                    u32x4 ip = {0, 0, 0, 0}; f32x4 w = {0, 0, 0, 0}; u8x4 dl = {0, 0, 0, 0};
                    if(inRow) {
                        ip = *reinterpret_cast<GLOBAL_AS const u32x4*>(ind + rowBase + j);
                        w = *reinterpret_cast<GLOBAL_AS const f32x4*>(weight + rowBase + j);
                        dl = *reinterpret_cast<GLOBAL_AS const u8x4*>(delay + rowBase + j);
                    }
                    const uint32_t s0 = (denPtr + dl.x) % D, s1 = (denPtr + dl.y) % D, s2 = (denPtr + dl.z) % D, s3 = (denPtr + dl.w) % D;
                    const bool skip = (G.skipZeroDelay != 0);       // slot == denPtr <=> d % D == 0
                    if(j < npost && !(skip && s0 == denPtr)) { atomicAddF32(&denDelay[(size_t)s0 * numTrg + ip.x], w.x); }
                    if(j + 1 < npost && !(skip && s1 == denPtr)) { atomicAddF32(&denDelay[(size_t)s1 * numTrg + ip.y], w.y); }
                    if(j + 2 < npost && !(skip && s2 == denPtr)) { atomicAddF32(&denDelay[(size_t)s2 * numTrg + ip.z], w.z); }
                    if(j + 3 < npost && !(skip && s3 == denPtr)) { atomicAddF32(&denDelay[(size_t)s3 * numTrg + ip.w], w.w); }
                }
                else {
                    uint32_t ip = 0; float w = 0; uint32_t dl = 0;
                    if(inRow) { ip = ind[rowBase + j]; w = weight[rowBase + j]; dl = delay[rowBase + j]; }
                    const uint32_t slot = (denPtr + dl) % D;
                    if(j < npost && !(G.skipZeroDelay && slot == denPtr)) { atomicAddF32(&denDelay[(size_t)slot * numTrg + ip], w); }
                }
            }
            else if(g.wum == GENNMI_WUM_STATIC_PULSE_REVERSE) {
                // addToPre(g): the weights of the row go to the spiking neuron itself; a lane sums its share, the lanes of the
                // (spike, chunk) item combine theirs, one atomic per item
                float sum = 0.0f;
                for(uint32_t q = 0; q < perLane; q++) { if(inRow && j + q < npost) { sum += weight[rowBase + j + q]; } }
                for(uint32_t off = W / 2; off > 0; off >>= 1) { sum += __shfl_xor(sum, off, WAVE); }
                if(lis == 0 && sum != 0.0f) { atomicAddF32(asGlobal(g.outPre) + (size_t)batch * g.numSrcNeurons + idPre, sum); }
            }
            else if(g.wum == GENNMI_WUM_STATIC_GRADED) {
                // event code of weightUpdateModels.h:318: addToPost(fmax(0.0, g * tanh((V_pre - Epre) / Vslope) * dt)).  The CPU
                // backend's generated code evaluates tanh, the products and the maximum in double (only the double versions of
                // tanh and fmax are in scope there); so does this, rounding once before the fp32 atomic.
                const float vPre = asGlobal(g.srcV)[(size_t)batch * g.numSrcNeurons + idPre];
                const double release = tanh((double)((vPre - g.gradedEpre) / g.gradedVslope));
                for(uint32_t q = 0; q < perLane; q++) {
                    if(inRow && j + q < npost) {
                        atomicAddF32(&outPost[ind[rowBase + j + q]], (float)fmax(0.0, (double)weight[rowBase + j + q] * release * (double)dt));
                    }
                }
            }
            else if(j < npost) {
                // trace STDP presynaptic-spike code (pygenn/genn_model.py:1456-1463); every synapse of
                // the row is owned by exactly one lane, so the read-modify-write of g needs no atomic
                const uint32_t idPost = ind[rowBase + j];
                const float w = weight[rowBase + j];
                const float stPost = dt + asGlobal(g.trgST)[idPost];   // st_post = DT*(backPropSteps+1) + trgST (synapseUpdateGroupMerged.cc:134-142)
                atomicAddF32(&outPost[idPost], w);
                const float dtSpike = st.t - stPost;
                if(dtSpike > 0) {
                    const float newWeight = w - (g.aMinus * asGlobal(g.postTrace)[idPost]);
                    weight[rowBase + j] = fminf(g.wMax, fmaxf(g.wMin, newWeight));
                }
            }
            if(lis == 0 && chunk == 0) { events += npost; }
        }
    }

    // one counter update per wave
    for(int off = WAVE / 2; off > 0; off >>= 1) { events += __shfl_down(events, off, WAVE); }
    if((threadIdx.x & (WAVE - 1)) == 0 && events) { atomicAdd(eventCounter, events); }
}

// ------------------------------------------------------------------------------------------------
// DENSE and BITMASK projections (single_threaded_cpu/backend.cc:1985-2021 is the sequential definition).  One lane
// per postsynaptic neuron walks the spike queue: weights of a spike's row are lane-consecutive (DENSE: g[idPre*numTrg
// + idPost]) or one bit each (BITMASK, most significant bit first), so there is nothing to scatter and no atomic —
// a lane that owns its outPost element alone continues the sum from the value that is there, in queue order, which is
// the CPU backend's order bit for bit.  When several projections feed one outPost, or a step carries so many spikes
// that the queue is shared between several blocks, the lane's partial sum is added with one (lane-consecutive) atomic.
// ------------------------------------------------------------------------------------------------
struct DenseGroupDev
{
    gennmi_presynaptic_update_group_t g;
    uint32_t startBlock, numBlocks;     // numBlocks = column blocks x slices
    uint32_t exclusive;                 // no other projection adds to this outPost
    uint32_t slices;                    // blocks that may share the spike queue of one block of columns
};

constexpr uint32_t DENSE_SPIKES_PER_SLICE = 16;     // a step with fewer spikes than this per slice uses fewer slices

__global__ __launch_bounds__(BLOCK)
void presynapticDenseKernel(const DenseGroupDev * __restrict__ blocks, unsigned long long *eventCounter)
{
    const DenseGroupDev &G = blocks[blockIdx.x];
    const gennmi_presynaptic_update_group_t &g = G.g;
    const uint32_t batch = blockIdx.y;
    const uint32_t local = blockIdx.x - G.startBlock;
    const uint32_t slice = local % G.slices;
    const uint32_t j = (local / G.slices) * BLOCK + threadIdx.x;
    const uint32_t numSpikes = asGlobal(g.srcSpkCnt)[batch];
    // The queue is cut into as many contiguous pieces as there are slices with at least 16 spikes each; with one
    // piece the lane continues the sum from outPost itself (exact queue order), with more every piece adds its partial sum.
    const uint32_t active = min(G.slices, max(1u, numSpikes / DENSE_SPIKES_PER_SLICE));
    if(numSpikes == 0 || slice >= active) { return; }
    const uint32_t perSlice = (numSpikes + active - 1) / active;
    const uint32_t first = slice * perSlice, last = min(numSpikes, first + perSlice);
    if(first >= numSpikes) { return; }          // rounding up perSlice can leave the last pieces empty
    const bool continueSum = G.exclusive && active == 1;
    GLOBAL_AS const uint32_t *spk = asGlobal(g.srcSpk) + (size_t)batch * g.numSrcNeurons;
    GLOBAL_AS float *outPost = asGlobal(g.outPost) + (size_t)batch * g.numTrgNeurons;
    unsigned long long events = 0;
    if(j < g.numTrgNeurons) {
        float acc = continueSum ? outPost[j] : 0.0f;
        if(g.matrix == GENNMI_MATRIX_DENSE) {
            const bool constant = (g.wum == GENNMI_WUM_STATIC_PULSE_CONSTANT_WEIGHT);
            GLOBAL_AS const float *weight = asGlobal(g.g);
            // eight rows in flight; the additions keep queue order
            uint32_t s = first;
            for(; s + 8 <= last; s += 8) {
                float w[8];
                #pragma unroll
                for(int u = 0; u < 8; u++) { w[u] = constant ? g.constantWeight : weight[(size_t)spk[s + u] * g.numTrgNeurons + j]; }
                #pragma unroll
                for(int u = 0; u < 8; u++) { acc += w[u]; }
            }
            for(; s < last; s++) { acc += constant ? g.constantWeight : weight[(size_t)spk[s] * g.numTrgNeurons + j]; }
            if(j == 0) { events = (unsigned long long)(last - first) * g.numTrgNeurons; }
        }
        else {
            GLOBAL_AS const uint32_t *gp = asGlobal(g.gp);
            for(uint32_t s = first; s < last; s++) {
                const unsigned long long gid = (unsigned long long)spk[s] * g.rowStride + j;
                if(gp[gid >> 5] & (0x80000000u >> (gid & 31))) { acc += g.constantWeight; events++; }
            }
        }
        if(continueSum) { outPost[j] = acc; }
        else if(acc != 0.0f) { atomicAddF32(&outPost[j], acc); }
    }
    for(int off = WAVE / 2; off > 0; off >>= 1) { events += __shfl_down(events, off, WAVE); }
    if((threadIdx.x & (WAVE - 1)) == 0 && events) { atomicAdd(eventCounter, events); }
}

// ------------------------------------------------------------------------------------------------
// PROCEDURAL connectivity (the reference's PostSpan/PreSpan procedural strategies, presynapticUpdateStrategySIMT.cc:391-560,
// re-run the connectivity snippet with a per-row generator state).  Here a wavefront regenerates the row of a spiking
// neuron with exactly the code and draws the initialisation kernels use (genn_mi355x_rows.h), so a procedural projection
// behaves synapse for synapse like the stored matrix the same seed would have produced — without reading a byte of
// connectivity: the only memory traffic of an event is its atomic.
// ------------------------------------------------------------------------------------------------
struct ProcGroupDev
{
    gennmi_presynaptic_update_group_t g;
    uint32_t startBlock, numBlocks;
    gennmi_rows::Stream connectivity, weight;
    gennmi_rows::VarInit weightInit;
    float probLogRecip;
    uint32_t pad_;
};

__global__ __launch_bounds__(BLOCK)
void presynapticProceduralKernel(const ProcGroupDev * __restrict__ blocks, unsigned long long *eventCounter)
{
    using namespace gennmi_rows;
    constexpr uint32_t MAX_ROUNDS = 64;                 // rows of up to 16,383 targets are shared between the block's waves
    __shared__ double shRoundTotal[MAX_ROUNDS];
    const ProcGroupDev &G = blocks[blockIdx.x];
    const gennmi_presynaptic_update_group_t &g = G.g;
    const uint32_t batch = blockIdx.y;
    const uint32_t lane = threadIdx.x & (WAVE - 1);
    const uint32_t wave = threadIdx.x / WAVE;
    const uint32_t localBlock = blockIdx.x - G.startBlock;
    const uint32_t numSpikes = asGlobal(g.srcSpkCnt)[batch];
    GLOBAL_AS const uint32_t *spk = asGlobal(g.srcSpk) + (size_t)batch * g.numSrcNeurons;
    GLOBAL_AS float *outPost = asGlobal(g.outPost) + (size_t)batch * g.numTrgNeurons;
    const uint32_t rowStride = g.rowStride;
    unsigned long long events = 0;
    if(g.procedural.connectivity == GENNMI_CONNECT_FIXED_NUMBER_POST) {
        const uint32_t n = min(g.procedural.num, rowStride);
        // a group of four synapses shares one generator call for its weights when the row starts on a multiple of four
        const bool aligned = (rowStride & 3u) == 0;
        auto deliver = [&](unsigned long long firstElement, uint32_t k, const uint32_t post[4]) {
            float w[4];
            if(aligned) { valuesAt4(G.weightInit, G.weight, firstElement + k, w); }
            else { for(int i = 0; i < 4; i++) { w[i] = valueAt(G.weightInit, G.weight, firstElement + k + i); } }
            for(int i = 0; i < 4 && k + i < n; i++) { atomicAddF32(&outPost[post[i]], w[i]); }
        };
        if(n / (4 * WAVE) + 1 > 1 && n / (4 * WAVE) + 1 <= MAX_ROUNDS) {
            // long rows: one spike per block, the block's waves share the row's rounds of 256 draws
            for(uint32_t s = localBlock; s < numSpikes; s += G.numBlocks) {
                const uint32_t row = spk[s];
                const unsigned long long firstElement = (unsigned long long)row * rowStride;
                fixedNumberPostRowBlock<BLOCK / WAVE>(row, g.numTrgNeurons, n, G.connectivity, lane, wave, shRoundTotal, MAX_ROUNDS,
                                                      [&](uint32_t k, const uint32_t post[4]) { deliver(firstElement, k, post); });
                if(threadIdx.x == 0) { events += n; }
            }
        }
        else {
            const uint32_t numWaves = G.numBlocks * (BLOCK / WAVE);
            for(uint32_t s = localBlock * (BLOCK / WAVE) + wave; s < numSpikes; s += numWaves) {
                const uint32_t row = spk[s];
                const unsigned long long firstElement = (unsigned long long)row * rowStride;
                fixedNumberPostRow(row, g.numTrgNeurons, n, G.connectivity, lane, [&](uint32_t k, const uint32_t post[4]) { deliver(firstElement, k, post); });
                if(lane == 0) { events += n; }
            }
        }
    }
    else {
        const uint32_t numWaves = G.numBlocks * (BLOCK / WAVE);
        for(uint32_t s = localBlock * (BLOCK / WAVE) + wave; s < numSpikes; s += numWaves) {
            const uint32_t row = spk[s];
            const unsigned long long firstElement = (unsigned long long)row * rowStride;
            const uint32_t total = fixedProbabilityRow(row, g.numTrgNeurons, G.probLogRecip,
                                                       g.procedural.connectivity == GENNMI_CONNECT_FIXED_PROBABILITY_NO_AUTAPSE, G.connectivity, lane,
                                                       [&](uint32_t k, uint32_t post) {
                if(k < rowStride) { atomicAddF32(&outPost[post], valueAt(G.weightInit, G.weight, firstElement + k)); }
            });
            if(lane == 0) { events += min(total, rowStride); }
        }
    }
    for(int off = WAVE / 2; off > 0; off >>= 1) { events += __shfl_down(events, off, WAVE); }
    if(lane == 0 && events) { atomicAdd(eventCounter, events); }
}

// ------------------------------------------------------------------------------------------------
// Tile kernel.  Scattered fp32 atomics cost one memory transaction each (≈20 G/s measured on this part,
// whatever the array size), lane-consecutive ones ≈280 G/s.  When a step carries enough events
// (numSpikes*rowStride >= numTrg), a block therefore owns a tile of postsynaptic neurons in LDS: it walks
// its share of the spike list, reads only the segment of each row that falls into its tile (rows are
// sorted by target; tileOff holds the segment boundaries), adds into LDS, and finally flushes the tile
// with consecutive lanes on consecutive addresses.
// ------------------------------------------------------------------------------------------------
__global__ __launch_bounds__(1024)
void presynapticTileKernel(const TileGroupDev * __restrict__ blocks, StepArgs args, float dt, unsigned long long *eventCounter)
{
    extern __shared__ float shTile[];
    const TileGroupDev &G = blocks[blockIdx.x];
    const gennmi_presynaptic_update_group_t &g = G.g;
    const uint32_t batch = blockIdx.y;
    const uint32_t numSpikes = asGlobal(g.srcSpkCnt)[batch];
    if((unsigned long long)numSpikes * g.rowStride < G.threshold) { return; }      // the scatter kernel took this step
    const uint32_t tileStart = G.tile * G.tileSize;
    const uint32_t tileLen = min(G.tileSize, g.numTrgNeurons - tileStart);
    for(uint32_t k = threadIdx.x; k < tileLen; k += blockDim.x) { shTile[k] = 0.0f; }
    __syncthreads();

    GLOBAL_AS const uint32_t *spk = asGlobal(g.srcSpk) + (size_t)batch * g.numSrcNeurons;
    GLOBAL_AS const uint16_t *off = asGlobal(G.tileOff);
    GLOBAL_AS const uint32_t *ind = asGlobal(g.ind);
    GLOBAL_AS float *weight = asGlobal(g.g);
    // trace-STDP rows: besides delivering the (old) weight, every event applies the presynaptic-spike rule to its own
    // synapse (pygenn/genn_model.py:1456-1463); a synapse belongs to exactly one tile, so g needs no atomic here either
    const bool stdp = (g.wum == GENNMI_WUM_STDP_TRACE);
    const float t = stdp ? resolve(args, dt).t : 0.0f;
    GLOBAL_AS const float *trgST = asGlobal(g.trgST);
    GLOBAL_AS const float *postTrace = asGlobal(g.postTrace);
    auto depress = [&](uint32_t idPost, float w) -> float {
        const float stPost = dt + trgST[idPost];
        const float dtSpike = t - stPost;
        if(dtSpike > 0) { return fminf(g.wMax, fmaxf(g.wMin, w - (g.aMinus * postTrace[idPost]))); }
        return w;
    };
    const uint32_t L = G.lanes;
    const uint32_t lis = threadIdx.x & (L - 1);
    const uint32_t perBlock = blockDim.x / L;
    const uint32_t stride = perBlock * G.numSplits;
    const uint32_t lastSrc = g.numSrcNeurons - 1;
    unsigned long long events = 0;
    // software pipeline over this sub-group's spikes: the spike id is fetched two iterations ahead and the
    // segment boundaries one iteration ahead (spk holds numSrcNeurons entries, so clamped indices are readable)
    uint32_t s = G.split * perBlock + threadIdx.x / L;
    uint32_t id0 = spk[min(s, lastSrc)], id1 = spk[min(s + stride, lastSrc)];
    size_t o0 = (size_t)id0 * (G.numTiles + 1) + G.tile;
    uint32_t a0 = off[o0], b0 = off[o0 + 1];
    for(; s < numSpikes; s += stride) {
        const uint32_t idPre = id0, a = a0, b = b0;
        id0 = id1;
        id1 = spk[min(s + 2 * stride, lastSrc)];
        o0 = (size_t)id0 * (G.numTiles + 1) + G.tile;
        a0 = off[o0]; b0 = off[o0 + 1];
        const size_t rowBase = (size_t)idPre * g.rowStride;
        for(uint32_t j = a + 4 * lis; j < b; j += 4 * L) {
            if(j + 4 <= b) {
                const u32x4u ip = *reinterpret_cast<GLOBAL_AS const u32x4u*>(ind + rowBase + j);
                const f32x4u w = *reinterpret_cast<GLOBAL_AS const f32x4u*>(weight + rowBase + j);
                if(stdp) {
                    f32x4u nw;
                    nw.x = depress(ip.x, w.x); nw.y = depress(ip.y, w.y); nw.z = depress(ip.z, w.z); nw.w = depress(ip.w, w.w);
                    *reinterpret_cast<GLOBAL_AS f32x4u*>(weight + rowBase + j) = nw;
                }
                unsafeAtomicAdd(&shTile[ip.x - tileStart], w.x);
                unsafeAtomicAdd(&shTile[ip.y - tileStart], w.y);
                unsafeAtomicAdd(&shTile[ip.z - tileStart], w.z);
                unsafeAtomicAdd(&shTile[ip.w - tileStart], w.w);
            }
            else {
                for(uint32_t jj = j; jj < b; jj++) {
                    const uint32_t idPost = ind[rowBase + jj];
                    const float w = weight[rowBase + jj];
                    if(stdp) { weight[rowBase + jj] = depress(idPost, w); }
                    unsafeAtomicAdd(&shTile[idPost - tileStart], w);
                }
            }
        }
        if(lis == 0) { events += b - a; }
    }
    __syncthreads();
    GLOBAL_AS float *outPost = asGlobal(g.outPost) + (size_t)batch * g.numTrgNeurons + tileStart;
    for(uint32_t k = threadIdx.x; k < tileLen; k += blockDim.x) {
        const float v = shTile[k];
        if(v != 0.0f) { atomicAddF32(&outPost[k], v); }
    }
    for(int o2 = WAVE / 2; o2 > 0; o2 >>= 1) { events += __shfl_down(events, o2, WAVE); }
    if((threadIdx.x & (WAVE - 1)) == 0 && events) { atomicAdd(eventCounter, events); }
}

// Toeplitz Conv2D counterpart of the tile kernel: every block finds the run of spikes whose kernel footprint touches
// its output rows and accumulates their contributions in an LDS tile, each wavefront in its own band of columns.  The block owns its rows exclusively, so the flush is a plain read-modify-write without atomics.
__global__ __launch_bounds__(CONV_TILE_THREADS)
void presynapticConvTileKernel(const ConvTileDev * __restrict__ blocks, unsigned long long *eventCounter)
{
    extern __shared__ float shConv[];
    const ConvTileDev &G = blocks[blockIdx.x];
    const gennmi_presynaptic_update_group_t &g = G.g;
    const uint32_t batch = blockIdx.y;
    const int kh = g.conv[0], kw = g.conv[1], iw = g.conv[3], ic = g.conv[4];
    const int oh = g.conv[5], ow = g.conv[6], oc = g.conv[7];
    const uint32_t numDiag = (uint32_t)(kh * kw * oc);
    const uint32_t numSpikes = asGlobal(g.srcSpkCnt)[batch];
    if((unsigned long long)numSpikes * numDiag < G.threshold) { return; }      // the scatter kernel took this step
    const int row0 = (int)G.tileRow0;
    const int rows = min((int)G.rowsPerTile, oh - row0);
    const uint32_t tileLen = (uint32_t)(rows * ow * oc);
    const uint32_t kernelLen = (uint32_t)(kh * kw * ic * oc);
    float *tile = shConv;
    float *kern = tile + G.rowsPerTile * ow * oc;
    uint32_t *stage = reinterpret_cast<uint32_t*>(kern + kernelLen);
    __shared__ uint32_t shLo, shHi;
    if(threadIdx.x == 0) { shLo = 0u; shHi = 0u; }
    for(uint32_t k = threadIdx.x; k < tileLen; k += blockDim.x) { tile[k] = 0.0f; }
    for(uint32_t k = threadIdx.x; k < kernelLen; k += blockDim.x) { kern[k] = asGlobal(g.g)[k]; }
    __syncthreads();

    // The queue is in ascending neuron index, i.e. sorted by input row, so the spikes whose kernel footprint reaches
    // this block's output rows — input rows [row0 + bh - kh + 1, row0 + rows + bh) — form one contiguous run
    // [lo, hi): count the spikes in front of either bound.
    GLOBAL_AS const uint32_t *spk = asGlobal(g.srcSpk) + (size_t)batch * g.numSrcNeurons;
    const uint32_t lane = threadIdx.x & (WAVE - 1);
    const uint32_t wave = threadIdx.x / WAVE, numWaves = blockDim.x / WAVE;
    const int firstRow = row0 + G.convBH - kh + 1, endRow = row0 + rows + G.convBH;
    uint32_t below = 0, upto = 0;
    for(uint32_t s = threadIdx.x; s < numSpikes; s += blockDim.x) {
        const int myRow = (int)(spk[s] / ic) / iw;
        below += (myRow < firstRow) ? 1u : 0u;
        upto += (myRow < endRow) ? 1u : 0u;
    }
    for(int o2 = WAVE / 2; o2 > 0; o2 >>= 1) { below += __shfl_down(below, o2, WAVE); upto += __shfl_down(upto, o2, WAVE); }
    if(lane == 0) { atomicAdd(&shLo, below); atomicAdd(&shHi, upto); }
    __syncthreads();
    const uint32_t lo = shLo, hi = shHi;
    unsigned long long events = 0;
    // The run is staged in LDS (decoded to row / column / channel) CONV_TILE_SPIKES at a time.  LDS float atomics
    // retire about one lane per clock, so none are used: every wavefront owns a band of output columns, picks the
    // staged spikes whose footprint touches its band (64 tested at a time), and adds their contributions to its own
    // columns with plain read-modify-write.  Per output element the contributions arrive in queue order, the order of
    // the CPU backend's loop.
    const int colsPerWave = (ow + (int)numWaves - 1) / (int)numWaves;
    const int col0 = (int)wave * colsPerWave, col1 = min(ow, col0 + colsPerWave);
    for(uint32_t base = lo; base < hi; base += CONV_TILE_SPIKES) {
        const uint32_t count = min((uint32_t)CONV_TILE_SPIKES, hi - base);
        __syncthreads();
        for(uint32_t k = threadIdx.x; k < count; k += blockDim.x) {
            const uint32_t id = spk[base + k];
            const uint32_t preRow = (id / ic) / iw, preCol = (id / ic) % iw, preChan = id % ic;
            // a queue that is not sorted would put foreign spikes inside the run: they are marked and skipped
            const bool relevant = ((int)preRow >= firstRow) && ((int)preRow < endRow);
            stage[k] = relevant ? (preRow << 20 | preCol << 10 | preChan) : 0xFFFFFFFFu;
        }
        __syncthreads();
        for(uint32_t sb = 0; sb < count && col0 < col1; sb += WAVE) {
            const uint32_t mine = (sb + lane < count) ? stage[sb + lane] : 0xFFFFFFFFu;
            const int myCol = (int)((mine >> 10) & 1023) - G.convBW;       // first output column this spike reaches
            unsigned long long pending = __ballot(mine != 0xFFFFFFFFu && myCol + kw - 1 >= col0 && myCol < col1);
            while(pending) {
                const int src = __ffsll((long long)pending) - 1;
                pending &= pending - 1;
                // everything about the spike and the kernel position is wavefront-uniform (scalar registers, scalar
                // branches); only the output channels are spread over the lanes
                const uint32_t pre = __builtin_amdgcn_readlane(mine, src);
                const int preRow = (int)(pre >> 20), preCol = (int)((pre >> 10) & 1023), preChan = (int)(pre & 1023);
                for(int kernRow = 0; kernRow < kh; kernRow++) {
                    const int postRow = preRow + kernRow - G.convBH;
                    if(postRow < row0 || postRow >= row0 + rows) { continue; }
                    for(int kernCol = 0; kernCol < kw; kernCol++) {
                        const int postCol = preCol + kernCol - G.convBW;
                        if(postCol < col0 || postCol >= col1) { continue; }
                        const float *weights = kern + (((kh - kernRow - 1) * kw + (kw - kernCol - 1)) * ic + preChan) * oc;
                        float *target = tile + ((postRow - row0) * ow + postCol) * oc;
                        for(int ch = (int)lane; ch < oc; ch += WAVE) { target[ch] += weights[ch]; }
                        if(lane == 0) { events += (unsigned long long)oc; }
                    }
                }
            }
        }
    }
    __syncthreads();
    GLOBAL_AS float *outPost = asGlobal(g.outPost) + (size_t)batch * g.numTrgNeurons + (size_t)row0 * ow * oc;
    // the block owns these rows, so plain read-modify-write; loads of a batch of elements are issued together
    for(uint32_t k0 = 0; k0 < tileLen; k0 += 8 * blockDim.x) {
        float old[8];
        #pragma unroll
        for(int u = 0; u < 8; u++) { const uint32_t k = k0 + u * blockDim.x + threadIdx.x; old[u] = (k < tileLen) ? outPost[k] : 0.0f; }
        #pragma unroll
        for(int u = 0; u < 8; u++) {
            const uint32_t k = k0 + u * blockDim.x + threadIdx.x;
            if(k < tileLen) { const float v = tile[k]; if(v != 0.0f) { outPost[k] = old[u] + v; } }
        }
    }
    for(int o2 = WAVE / 2; o2 > 0; o2 >>= 1) { events += __shfl_down(events, o2, WAVE); }
    if(lane == 0 && events) { atomicAdd(eventCounter, events); }
}

// Segment boundaries of every row for the tile kernel; also verifies that rows are sorted by target.
__global__ void tileOffsetKernel(uint32_t numSrc, uint32_t rowStride, const uint32_t *rowLength, const uint32_t *ind,
                                 uint32_t tileSize, uint32_t numTiles, uint16_t *off, uint32_t *unsorted)
{
    const uint32_t row = blockIdx.x * blockDim.x + threadIdx.x;
    if(row >= numSrc) { return; }
    const uint32_t len = rowLength[row];
    const uint32_t *r = ind + (size_t)row * rowStride;
    uint16_t *o = off + (size_t)row * (numTiles + 1);
    uint32_t t = 0, prev = 0;
    for(uint32_t j = 0; j < len; j++) {
        const uint32_t p = r[j];
        if(p < prev) { atomicOr(unsorted, 1u); }
        prev = p;
        while(t <= numTiles && (unsigned long long)t * tileSize <= p) { o[t++] = (uint16_t)j; }
    }
    while(t <= numTiles) { o[t++] = (uint16_t)len; }
}

__global__ __launch_bounds__(BLOCK)
void presynapticUpdateKernel(const PreGroupDev * __restrict__ blocks, StepArgs args, float dt, unsigned long long *eventCounter)
{
    presynapticBody(blocks[blockIdx.x], blockIdx.x, resolve(args, dt), dt, eventCounter);
}

// ------------------------------------------------------------------------------------------------
// Postsynaptic update (learnPost): one sub-group per postsynaptic spike walks the column through
// remap (coalesced), gathers g by synapse index.
// ------------------------------------------------------------------------------------------------
__global__ __launch_bounds__(BLOCK)
void postsynapticUpdateKernel(const PostGroupDev * __restrict__ blocks, StepArgs args, float dt)
{
    const Resolved st = resolve(args, dt);
    const PostGroupDev &G = blocks[blockIdx.x];
    const gennmi_postsynaptic_update_group_t &g = G.g;
    const uint32_t W = G.lanesPerSpike;
    const uint32_t localBlock = blockIdx.x - G.startBlock;
    const uint32_t lis = threadIdx.x & (W - 1);
    const uint32_t subGroup = (localBlock * BLOCK + threadIdx.x) / W;
    const uint32_t numSubGroups = (G.numBlocks * BLOCK) / W;
    const uint32_t numSpikes = g.trgSpkCnt[0];
    if(G.denseThreshold && numSpikes >= G.denseThreshold) {
        // A large share of the target population fired: nearly every row holds synapses to update, so walk the rows
        // once (coalesced ind / g) and test each synapse's target against the spike bitmap, instead of one scattered
        // read-modify-write per (spike, column entry).  Same arithmetic per synapse; every synapse is visited once.
        extern __shared__ uint32_t shBits[];
        const uint32_t words = (g.numTrgNeurons + 31) / 32;
        for(uint32_t k = threadIdx.x; k < words; k += BLOCK) { shBits[k] = asGlobal(G.spikeBitmap)[k]; }
        __syncthreads();
        const uint32_t lane = threadIdx.x & (WAVE - 1);
        const uint32_t numWaves = G.numBlocks * (BLOCK / WAVE);
        GLOBAL_AS const uint32_t *ind = asGlobal(g.ind);
        GLOBAL_AS float *weight = asGlobal(g.g);
        // per-row scalars of the NEXT row are fetched while the current one is processed (indices clamped: readable)
        const uint32_t lastRow = g.numSrcNeurons - 1;
        uint32_t row = localBlock * (BLOCK / WAVE) + threadIdx.x / WAVE;
        uint32_t lenNext = asGlobal(g.rowLength)[min(row, lastRow)];
        float stNext = asGlobal(g.srcST)[min(row, lastRow)], traceNext = asGlobal(g.preTrace)[min(row, lastRow)];
        for(; row < g.numSrcNeurons; row += numWaves) {
            const uint32_t len = lenNext;
            const float stPre = dt + stNext;
            const float step = g.aPlus * traceNext;
            const uint32_t nextRow = min(row + numWaves, lastRow);
            lenNext = asGlobal(g.rowLength)[nextRow]; stNext = asGlobal(g.srcST)[nextRow]; traceNext = asGlobal(g.preTrace)[nextRow];
            const float dtSpike = st.t - stPre;
            if(!(dtSpike > 0) || len == 0) { continue; }
            const size_t rowBase = (size_t)row * g.rowStride;
            // up to four strides of the row in flight per lane
            for(uint32_t j0 = lane; j0 < len; j0 += 4 * WAVE) {
                uint32_t idPost[4]; float w[4];
                #pragma unroll
                for(int u = 0; u < 4; u++) {
                    const uint32_t j = j0 + u * WAVE;
                    idPost[u] = (j < len) ? ind[rowBase + j] : 0xFFFFFFFFu;
                    w[u] = (j < len) ? weight[rowBase + j] : 0.0f;
                }
                #pragma unroll
                for(int u = 0; u < 4; u++) {
                    if(idPost[u] != 0xFFFFFFFFu && ((shBits[idPost[u] >> 5] >> (idPost[u] & 31)) & 1u)) {
                        weight[rowBase + j0 + u * WAVE] = fminf(g.wMax, fmaxf(g.wMin, w[u] + step));
                    }
                }
            }
        }
        return;
    }
    for(uint32_t s = subGroup; s < numSpikes; s += numSubGroups) {
        const uint32_t spike = g.trgSpk[s];
        const uint32_t npre = g.colLength[spike];
        const size_t colBase = (size_t)spike * g.colStride;
        for(uint32_t i = lis; i < npre; i += W) {
            const uint32_t rowMajorIndex = g.remap[colBase + i];
            const uint32_t idPre = rowMajorIndex / g.rowStride;
            const float stPre = dt + g.srcST[idPre];
            const float dtSpike = st.t - stPre;
            if(dtSpike > 0) {
                const float newWeight = g.g[rowMajorIndex] + (g.aPlus * g.preTrace[idPre]);
                g.g[rowMajorIndex] = fminf(g.wMax, fmaxf(g.wMin, newWeight));
            }
        }
    }
}

// ------------------------------------------------------------------------------------------------
// Offset of a block's entries in its population's queue: the block publishes its count, then (wave 0) sums the counts of
// the earlier blocks of its group of 64 and the published totals of the earlier groups.  Every thread of the block calls
// this between two barriers of its own; returns 0xFFFFFFFF after a bounded wait expired (error flag raised).
__device__ __forceinline__ uint32_t blockQueueOffset(uint32_t blockCount, uint32_t localBlock, uint32_t numBlocks, size_t aggBase,
                                                    unsigned long long *counts, unsigned long long *groupTotals, uint32_t tag,
                                                    uint32_t *shOffset, uint32_t *errorFlag)
{
    const uint32_t lane = threadIdx.x & (WAVE - 1);
    const uint32_t wave = threadIdx.x / WAVE;
    if(threadIdx.x == 0) {
        __hip_atomic_store(&counts[aggBase + localBlock], ((unsigned long long)tag << 32) | blockCount, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    const bool last = (localBlock == numBlocks - 1);
    if(wave == 0) {
        const uint32_t group = localBlock / WAVE, inGroup = localBlock % WAVE;
        const size_t groupBase = aggBase + (size_t)group * WAVE;
        bool ok = true;
        auto waitFor = [&](const unsigned long long *p) -> uint32_t {
            uint32_t spins = 0;
            while(true) {
                const unsigned long long a = __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                if((uint32_t)(a >> 32) == tag) { return (uint32_t)a; }
                if(++spins > c_spinLimit) { ok = false; return 0u; }
                __builtin_amdgcn_s_sleep(1);
            }
        };
        uint32_t intra = (lane < inGroup) ? waitFor(&counts[groupBase + lane]) : 0u;
        for(int off = WAVE / 2; off > 0; off >>= 1) { intra += __shfl_down(intra, off, WAVE); }
        intra = __shfl(intra, 0, WAVE);
        if((inGroup == WAVE - 1 || last) && lane == 0 && ok) {
            __hip_atomic_store(&groupTotals[aggBase + group], ((unsigned long long)tag << 32) | (intra + blockCount), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        uint32_t sum = 0;
        if(blockCount != 0 || last) {
            for(uint32_t base = 0; base < group; base += WAVE) {
                if(base + lane < group) { sum += waitFor(&groupTotals[aggBase + base + lane]); }
            }
            for(int off = WAVE / 2; off > 0; off >>= 1) { sum += __shfl_down(sum, off, WAVE); }
            sum += intra;
        }
        const bool allOk = (__ballot(!ok) == 0ull);
        if(lane == 0) {
            if(!allOk) { atomicOr(errorFlag, 1u); sum = 0xFFFFFFFFu; }
            *shOffset = sum;
        }
    }
    __syncthreads();
    return *shOffset;
}

// ------------------------------------------------------------------------------------------------
// Ordered append of the flagged neurons of a population to a queue, for spike-like events: the scheme the neuron
// update uses for true spikes (ballot rank in the wave, LDS scan in the block, look-back over per-block counts tagged
// with the step, blocks in groups of 64 with a published group total), as a function every block of the population
// calls with all its threads.  `counts` and `groupTotals` hold one entry per (batch, neuron block of the launch).
// ------------------------------------------------------------------------------------------------
__device__ __forceinline__ void appendOrdered(bool flag, uint32_t id, uint32_t localBlock, uint32_t numBlocks, size_t aggBase,
                                              unsigned long long *counts, unsigned long long *groupTotals, uint32_t tag,
                                              uint32_t *queue, uint32_t *queueCount, uint32_t *errorFlag,
                                              uint32_t *recordWords = nullptr, bool inRange = false)
{
    __shared__ uint32_t shCount[BLOCK / WAVE];
    __shared__ uint32_t shOffset;
    const uint32_t lane = threadIdx.x & (WAVE - 1);
    const uint32_t wave = threadIdx.x / WAVE;
    const unsigned long long ballot = __ballot(flag);
    // recording: the ballot is the bitfield of this step's events (every word of the step is overwritten)
    if(recordWords && (lane & 31) == 0 && inRange) { recordWords[id >> 5] = (uint32_t)(ballot >> (lane & 32)); }
    const uint32_t laneRank = __popcll(ballot & ((1ull << lane) - 1ull));
    if(lane == 0) { shCount[wave] = __popcll(ballot); }
    __syncthreads();
    uint32_t blockCount = 0, waveOffset = 0;
    #pragma unroll
    for(uint32_t w = 0; w < BLOCK / WAVE; w++) {
        const uint32_t c = shCount[w];
        if(w < wave) { waveOffset += c; }
        blockCount += c;
    }
    const uint32_t prefix = blockQueueOffset(blockCount, localBlock, numBlocks, aggBase, counts, groupTotals, tag, &shOffset, errorFlag);
    if(prefix != 0xFFFFFFFFu) {
        if(flag) { queue[prefix + waveOffset + laneRank] = id; }
        if(localBlock == numBlocks - 1 && threadIdx.x == 0) { *queueCount = prefix + blockCount; }
    }
    __syncthreads();            // the shared words are reused by the next call
}

// ------------------------------------------------------------------------------------------------
// Neuron update.  One lane per neuron.  Spikes are emitted in ascending neuron index (the CPU
// backend's order, single_threaded_cpu/backend.cc:321, 2119-2133): wave ballot gives the in-wave
// rank, an LDS scan the in-block rank, and a look-back over per-block counts published in `agg`
// (tagged with the step so nothing ever needs clearing) the cross-block offset.  Only blocks that
// emitted spikes, and the last block of each population (which stores spkCnt), look back.
// ------------------------------------------------------------------------------------------------
__device__ __forceinline__ void neuronBody(const NeuronGroupDev &G, uint32_t blockInKernel, uint32_t totalNeuronBlocks,
                                           const Resolved &st, float dt, unsigned long long *agg, uint32_t *errorFlag)
{
    __shared__ uint32_t shWaveCount[BLOCK / WAVE];
    __shared__ uint32_t shPrefix;

    const gennmi_neuron_update_group_t &g = G.g;
    const uint32_t batch = blockIdx.y;
    const uint32_t localBlock = blockInKernel - G.startBlock;
    const uint32_t n = g.numNeurons;
    const uint32_t i = localBlock * BLOCK + threadIdx.x;
    const size_t bi = (size_t)batch * n + i;
    const uint32_t lane = threadIdx.x & (WAVE - 1);
    const uint32_t wave = threadIdx.x / WAVE;
    const float t = st.t;

    bool spiked = false;
    float vEvent = 0.0f;
    uint32_t z0 = 0, z1 = 0;
    if(G.zeroStart && i < n) { z0 = asGlobal(G.zeroStart)[i]; z1 = asGlobal(G.zeroStart)[i + 1]; }
    if(i < n) {
        // order of operations: neuronUpdateGroupMerged.cc:552-773 — PSMs, current sources, sim code,
        // WU pre/post dynamics, threshold, then (on a spike) WU pre/post spike code, sT, reset
        float l0 = 0, l1 = 0;
        uint32_t startSpike = 0;
        float nextTime = 0.0f;
        if(g.model == GENNMI_NEURON_SPIKE_SOURCE_ARRAY) {
            // one coalesced read instead of startSpike, endSpike and a gather from spikeTimes: the time of the neuron's next
            // spike is kept beside the state and refreshed only when the neuron fires
            nextTime = asGlobal(G.nextSpikeTime)[bi];
        }
        else {
            // Every load of this neuron's inputs is issued before the first store: the pointers come out of a
            // descriptor in memory, so a store in between would force the compiler to re-read the descriptor
            // and would serialise the loads, and each dependent access costs about a microsecond at the start of
            // a launch (nothing is cached yet).  Sums keep the reference's order (PSMs, then current sources).
            float lin[GENNMI_MAX_PSM], front[GENNMI_MAX_PSM], inj[GENNMI_MAX_CS], rev[GENNMI_MAX_PRE_OUTPUT];
            const uint32_t numPSM = g.numPSM, numCS = g.numCS, numRev = g.numPreOutput;
            #pragma unroll
            for(uint32_t q = 0; q < GENNMI_MAX_PRE_OUTPUT; q++) { rev[q] = (q < numRev) ? asGlobal(g.outPre[q])[bi] : 0.0f; }
            l0 = asGlobal(g.var0)[bi]; l1 = asGlobal(g.var1)[bi];
            #pragma unroll
            for(uint32_t m = 0; m < GENNMI_MAX_PSM; m++) {
                lin[m] = 0.0f; front[m] = 0.0f;
                if(m < numPSM) {
                    lin[m] = asGlobal(g.psm[m].outPost)[bi];
                    const uint32_t D = g.psm[m].maxDenDelay;
                    if(D) { front[m] = asGlobal(g.psm[m].denDelay)[((size_t)batch * D + modStep(st.epoch + 1, D)) * n + i]; }
                }
            }
            #pragma unroll
            for(uint32_t c = 0; c < GENNMI_MAX_CS; c++) {
                inj[c] = 0.0f;
                if(c < numCS) {
                    inj[c] = (g.cs[c].kind == GENNMI_CS_DC) ? g.cs[c].amp
                                                            : asGlobal(g.cs[c].array)[(size_t)modStep(st.epoch, g.cs[c].arraySteps) * n + i];
                }
            }
            float Isyn = 0;
            #pragma unroll
            for(uint32_t m = 0; m < GENNMI_MAX_PSM; m++) {
                if(m < numPSM) {
                    // read and clear the front slot of the ring (neuronUpdateGroupMerged.cc:84-101)
                    float linSyn = lin[m];
                    const uint32_t D = g.psm[m].maxDenDelay;
                    if(D) { linSyn += front[m]; }
                    if(g.psm[m].kind == GENNMI_PSM_EXPCURR) {
                        Isyn += g.psm[m].init * linSyn;
                        linSyn *= g.psm[m].expDecay;
                    }
                    else {
                        Isyn += linSyn;
                        linSyn = 0.0f;
                    }
                    lin[m] = linSyn;
                }
            }
            // presynaptic output of the outgoing projections: after the postsynaptic models, before the current sources
            #pragma unroll
            for(uint32_t q = 0; q < GENNMI_MAX_PRE_OUTPUT; q++) { if(q < numRev) { Isyn += rev[q]; } }
            #pragma unroll
            for(uint32_t c = 0; c < GENNMI_MAX_CS; c++) { if(c < numCS) { Isyn += inj[c]; } }
            #pragma unroll
            for(uint32_t q = 0; q < GENNMI_MAX_PRE_OUTPUT; q++) { if(q < numRev) { asGlobal(g.outPre[q])[bi] = 0.0f; } }
            #pragma unroll
            for(uint32_t m = 0; m < GENNMI_MAX_PSM; m++) {
                if(m < numPSM) {
                    const uint32_t D = g.psm[m].maxDenDelay;
                    if(D) { asGlobal(g.psm[m].denDelay)[((size_t)batch * D + modStep(st.epoch + 1, D)) * n + i] = 0.0f; }
                    asGlobal(g.psm[m].outPost)[bi] = lin[m];
                }
            }
            if(g.model == GENNMI_NEURON_LIF) {
                if(l1 <= 0.0f) {
                    const float alpha = ((Isyn + g.params[0]) * g.params[1]) + g.params[2];
                    l0 = alpha - (g.params[3] * (alpha - l0));
                }
                else {
                    l1 -= dt;
                }
            }
            else {
                if(l0 >= 30.0f) {
                    l0 = g.params[2];
                    l1 += g.params[3];
                }
                l0 += 0.5f * (0.04f * l0 * l0 + 5.0f * l0 + 140.0f - l1 + Isyn) * dt;
                l0 += 0.5f * (0.04f * l0 * l0 + 5.0f * l0 + 140.0f - l1 + Isyn) * dt;
                l1 += g.params[0] * (g.params[1] * l0 - l1) * dt;
                if(l0 > 30.0f) { l0 = 30.0f; }
            }
        }
        float preTrace = 0, postTrace = 0;
        if(g.preTrace) { preTrace = g.preTrace[bi] * g.preDecay; }
        if(g.postTrace) { postTrace = g.postTrace[bi] * g.postDecay; }
        if(g.model == GENNMI_NEURON_LIF) { spiked = (l1 <= 0.0f && l0 >= g.params[4]); }
        else if(g.model == GENNMI_NEURON_IZHIKEVICH) { spiked = (l0 >= 29.99f); }
        else { spiked = (t >= nextTime); }       // startSpike != endSpike && t >= spikeTimes[startSpike] (neuronModels.h:274-286)
        vEvent = l0;           // spike-like event conditions see the updated V before any reset (neuronUpdateGroupMerged.cc:677-683)
        if(spiked) {
            preTrace += 1.0f; postTrace += 1.0f;
            if(g.sT) { g.sT[bi] = t; }
            if(g.model == GENNMI_NEURON_LIF) { l0 = g.params[5]; l1 = g.params[6]; }
            else if(g.model == GENNMI_NEURON_SPIKE_SOURCE_ARRAY) {
                startSpike = g.startSpike[bi] + 1;
                g.startSpike[bi] = startSpike;
                G.nextSpikeTime[bi] = (startSpike != g.endSpike[bi]) ? g.spikeTimes[startSpike] : INFINITY;
            }
        }
        if(g.preTrace) { g.preTrace[bi] = preTrace; }
        if(g.postTrace) { g.postTrace[bi] = postTrace; }
        if(g.model != GENNMI_NEURON_SPIKE_SOURCE_ARRAY) { g.var0[bi] = l0; g.var1[bi] = l1; }
    }

    // keep the user-visible ring pointers current (nothing in the kernels reads them)
    if(localBlock == 0 && batch == 0 && threadIdx.x < g.numPSM) {
        const gennmi_psm_t &psm = g.psm[threadIdx.x];
        if(psm.maxDenDelay && psm.denDelayPtr) { *psm.denDelayPtr = modStep(st.epoch + 1, psm.maxDenDelay); }
    }

    // ---- spike-like events: one ordered queue per event condition ----------------------------------
    if(g.numSpkEvent) {
        const size_t perArea = (size_t)totalNeuronBlocks * gridDim.y;
        for(uint32_t e = 0; e < g.numSpkEvent; e++) {
            unsigned long long *counts = G.aggEvent + (size_t)e * 2 * perArea;
            appendOrdered(i < n && vEvent > g.spkEvent[e].threshold, i, localBlock, G.numBlocks, (size_t)batch * totalNeuronBlocks + G.startBlock,
                          counts, counts + perArea, (uint32_t)(st.epoch + 1), g.spkEvent[e].spkEvent + (size_t)batch * n,
                          g.spkEvent[e].spkCntEvent + batch, errorFlag,
                          g.spkEvent[e].recordSpkEvent ? g.spkEvent[e].recordSpkEvent + ((size_t)st.recT * gridDim.y + batch) * ((n + 31) / 32) : nullptr, i < n);
        }
    }

    // ---- ordered compaction --------------------------------------------------------------------
    const unsigned long long ballot = __ballot(spiked);
    const uint32_t waveCount = __popcll(ballot);
    const uint32_t laneRank = __popcll(ballot & ((1ull << lane) - 1ull));
    if(lane == 0) { shWaveCount[wave] = waveCount; }

    // recording: the ballot IS the bitfield (bit i%32 of word i/32, runtime.cc:855-913); every word of
    // the step is overwritten, so no clearing and no atomicOr (cf. backendSIMT.cc:1948-1953)
    if(g.recordSpk && (lane & 31) == 0 && i < n) {
        const uint32_t words = (n + 31) / 32;
        g.recordSpk[((size_t)st.recT * gridDim.y + batch) * words + (i >> 5)] = (uint32_t)(ballot >> (lane & 32));
    }
    if(G.spikeBitmap && (lane & 31) == 0 && i < n) { G.spikeBitmap[i >> 5] = (uint32_t)(ballot >> (lane & 32)); }
    __syncthreads();

    uint32_t blockCount = 0, waveOffset = 0;
    #pragma unroll
    for(uint32_t w = 0; w < BLOCK / WAVE; w++) {
        const uint32_t c = shWaveCount[w];
        if(w < wave) { waveOffset += c; }
        blockCount += c;
    }

    const uint32_t tag = (uint32_t)(st.epoch + 1);
    const size_t aggBase = (size_t)batch * totalNeuronBlocks + G.startBlock;
    if(threadIdx.x == 0) {
        // the count itself is all that is communicated, so a relaxed device-scope store suffices
        // (release would write back the whole L2 from every block)
        __hip_atomic_store(&agg[aggBase + localBlock], ((unsigned long long)tag << 32) | blockCount,
                           __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    const bool last = (localBlock == G.numBlocks - 1);
    const bool groupLeader = ((localBlock % WAVE) == WAVE - 1) || last;
    if(blockCount == 0 && !groupLeader) { return; }

    // Synapses with d % D == 0 of the neurons that just fired belong in the slot their targets read in the
    // NEXT step, (epoch + 2) % D, which nothing reads or clears during this step — so the presynaptic update of
    // the next step (which skips them) may run concurrently with that step's neuron update.  The wavefront
    // delivers them cooperatively, one fired neuron at a time, lanes striding over its merged list.
    auto deliverZeroDelay = [&]() {
        unsigned long long pending = ballot;
        while(pending) {
            const int src = __ffsll((long long)pending) - 1;
            pending &= pending - 1;
            const uint32_t s0 = __shfl(z0, src, WAVE), s1 = __shfl(z1, src, WAVE);
            for(uint32_t k = s0 + lane; k < s1; k += WAVE) {
                const ZeroDelayEntry e = G.zeroEntries[k];
                const uint32_t slot = modStep(st.epoch + 2, e.maxDenDelay);
                atomicAddF32(asGlobal(e.ringElem) + ((size_t)batch * e.maxDenDelay + slot) * e.numTrgNeurons, *asGlobal(e.weight));
            }
        }
    };
    if(G.zeroStart && wave != 0) { deliverZeroDelay(); }

    if(wave == 0) {
        // Two-level offset: blocks of a population form groups of 64.  The last block of a group sums the
        // group's 64 counts and publishes the group total in the second half of `agg`; a block's offset is the
        // sum of the counts of the earlier blocks of its group plus the totals of the earlier groups.  Every
        // wait is for a value that depends only on other blocks having published their own count, so there is
        // no chain of blocks waiting for each other's results, whatever the population size.
        unsigned long long *groupAgg = agg + (size_t)totalNeuronBlocks * gridDim.y;
        const uint32_t group = localBlock / WAVE, inGroup = localBlock % WAVE;
        const size_t groupBase = aggBase + (size_t)group * WAVE;
        bool ok = true;
        auto waitFor = [&](const unsigned long long *p) -> uint32_t {
            uint32_t spins = 0;
            while(true) {
                const unsigned long long a = __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                if((uint32_t)(a >> 32) == tag) { return (uint32_t)a; }
                if(++spins > c_spinLimit) { ok = false; return 0u; }
                __builtin_amdgcn_s_sleep(1);
            }
        };
        // counts of the earlier blocks of this group (lane == inGroup contributes this block's own count)
        uint32_t v = 0;
        if(lane < inGroup) { v = waitFor(&agg[groupBase + lane]); }
        uint32_t intra = v;
        for(int off = WAVE / 2; off > 0; off >>= 1) { intra += __shfl_down(intra, off, WAVE); }
        intra = __shfl(intra, 0, WAVE);
        if(inGroup == WAVE - 1 || last) {
            if(lane == 0 && ok) {
                __hip_atomic_store(&groupAgg[aggBase + group], ((unsigned long long)tag << 32) | (intra + blockCount),
                                   __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
        }
        uint32_t sum = 0;
        if(blockCount != 0 || last) {
            for(uint32_t base = 0; base < group; base += WAVE) {
                if(base + lane < group) { sum += waitFor(&groupAgg[aggBase + base + lane]); }
            }
            for(int off = WAVE / 2; off > 0; off >>= 1) { sum += __shfl_down(sum, off, WAVE); }
            sum += intra;
        }
        const bool allOk = (__ballot(!ok) == 0ull);
        if(lane == 0) {
            if(!allOk) { atomicOr(errorFlag, 1u); sum = 0xFFFFFFFFu; }
            shPrefix = sum;
        }
    }
    __syncthreads();
    const uint32_t prefix = shPrefix;
    if(prefix == 0xFFFFFFFFu) { return; }       // bounded wait expired: flagged, nothing written
    // with axonal delay the queue is a ring of slots and this step writes slot (epoch + 1) % slots: the reference's
    // spkQuePtr after the increment at the start of its updateNeurons (neuronUpdateGroupMerged.cc:947-953)
    const uint32_t delaySlots = max(1u, g.numDelaySlots);
    const size_t queue = (size_t)batch * delaySlots + ((delaySlots > 1) ? modStep(st.epoch + 1, delaySlots) : 0u);
    if(spiked) { g.spk[queue * n + prefix + waveOffset + laneRank] = i; }
    if(last && threadIdx.x == 0) { g.spkCnt[queue] = prefix + blockCount; }
    // further copies of the queue (one population can feed several spike arrays: its own outgoing projections
    // and, for learnPost, the incoming plastic ones; runtime.cc:267-278)
    for(uint32_t q = 0; q < g.numExtraSpk; q++) {
        if(spiked) { g.extraSpk[q][(size_t)batch * n + prefix + waveOffset + laneRank] = i; }
        if(last && threadIdx.x == 0) { g.extraSpkCnt[q][batch] = prefix + blockCount; }
    }
    if(G.shadowSpk) {
        const uint32_t parity = (uint32_t)(st.epoch & 1);
        if(spiked) { G.shadowSpk[((size_t)parity * gridDim.y + batch) * n + prefix + waveOffset + laneRank] = i; }
        if(last && threadIdx.x == 0) { G.shadowCnt[(size_t)parity * gridDim.y + batch] = prefix + blockCount; }
    }
    if(G.zeroStart && wave == 0) { deliverZeroDelay(); }
}

__global__ __launch_bounds__(BLOCK)
void neuronUpdateKernel(const NeuronGroupDev * __restrict__ blocks, StepArgs args, float dt,
                        unsigned long long *agg, uint32_t *errorFlag)
{
    neuronBody(blocks[blockIdx.x], blockIdx.x, gridDim.x, resolve(args, dt), dt, agg, errorFlag);
}

// ------------------------------------------------------------------------------------------------
// Neuron update for large populations.  With one neuron per lane a population of millions is many rounds of resident
// work-groups, and every round pays the whole dependent chain (descriptor, inputs, count published, look-back, queue).
// Here a wavefront takes NPL consecutive chunks of 64 neurons: all inputs of all chunks are requested before anything is
// stored, so a lane has NPL times the bytes in flight and the launch has 1/NPL of the work-groups.  Same arithmetic per
// neuron and the same ordered queue as neuronBody (chunks of a wave are consecutive neurons, so chunk-major rank is neuron
// order); the subset of features large populations use: LIF, Izhikevich and spike-source groups with up to two
// postsynaptic models and one current source, spike recording; no traces, spike times, delay slots, further spike arrays,
// events or presynaptic output (the host picks this kernel only when every group fits).
// ------------------------------------------------------------------------------------------------
constexpr uint32_t BULK_MAX_PSM = 2, BULK_MAX_CS = 1;

template<int NPL>
__device__ __forceinline__ void neuronBulkBody(const NeuronGroupDev &G, uint32_t blockInKernel, uint32_t totalNeuronBlocks,
                                               const Resolved &st, float dt, unsigned long long *agg, uint32_t *errorFlag)
{
    __shared__ uint32_t shWaveCount[BLOCK / WAVE];
    __shared__ uint32_t shPrefix;
    const gennmi_neuron_update_group_t &g = G.g;
    const uint32_t batch = blockIdx.y;
    const uint32_t localBlock = blockInKernel - G.startBlock;
    const uint32_t n = g.numNeurons;
    const uint32_t lane = threadIdx.x & (WAVE - 1);
    const uint32_t wave = threadIdx.x / WAVE;
    const float t = st.t;
    const uint32_t first = (localBlock * (BLOCK / WAVE) + wave) * (WAVE * NPL) + lane;      // this lane's neuron in chunk 0
    const uint32_t numPSM = g.numPSM, numCS = g.numCS;

    float l0[NPL], l1[NPL], lin[NPL][BULK_MAX_PSM], front[NPL][BULK_MAX_PSM], inj[NPL];
    bool spiked[NPL];
    // ---- every input of every chunk first
    #pragma unroll
    for(int j = 0; j < NPL; j++) {
        const uint32_t i = first + j * WAVE;
        const size_t bi = (size_t)batch * n + i;
        l0[j] = l1[j] = inj[j] = 0.0f;
        #pragma unroll
        for(uint32_t m = 0; m < BULK_MAX_PSM; m++) { lin[j][m] = front[j][m] = 0.0f; }
        spiked[j] = false;
        if(i < n) {
            if(g.model == GENNMI_NEURON_SPIKE_SOURCE_ARRAY) {
                l0[j] = asGlobal(G.nextSpikeTime)[bi];
            }
            else {
                l0[j] = asGlobal(g.var0)[bi]; l1[j] = asGlobal(g.var1)[bi];
                #pragma unroll
                for(uint32_t m = 0; m < BULK_MAX_PSM; m++) {
                    if(m < numPSM) {
                        lin[j][m] = asGlobal(g.psm[m].outPost)[bi];
                        const uint32_t D = g.psm[m].maxDenDelay;
                        if(D) { front[j][m] = asGlobal(g.psm[m].denDelay)[((size_t)batch * D + modStep(st.epoch + 1, D)) * n + i]; }
                    }
                }
                if(numCS) {
                    inj[j] = (g.cs[0].kind == GENNMI_CS_DC) ? g.cs[0].amp
                                                            : asGlobal(g.cs[0].array)[(size_t)modStep(st.epoch, g.cs[0].arraySteps) * n + i];
                }
            }
        }
    }
    // ---- update and store, chunk by chunk (operations and their order as in neuronBody)
    #pragma unroll
    for(int j = 0; j < NPL; j++) {
        const uint32_t i = first + j * WAVE;
        const size_t bi = (size_t)batch * n + i;
        if(i >= n) { continue; }
        if(g.model == GENNMI_NEURON_SPIKE_SOURCE_ARRAY) {
            spiked[j] = (t >= l0[j]);
            if(spiked[j]) {
                const uint32_t startSpike = g.startSpike[bi] + 1;
                g.startSpike[bi] = startSpike;
                G.nextSpikeTime[bi] = (startSpike != g.endSpike[bi]) ? g.spikeTimes[startSpike] : INFINITY;
            }
            continue;
        }
        float Isyn = 0;
        #pragma unroll
        for(uint32_t m = 0; m < BULK_MAX_PSM; m++) {
            if(m < numPSM) {
                float linSyn = lin[j][m];
                const uint32_t D = g.psm[m].maxDenDelay;
                if(D) { linSyn += front[j][m]; }
                if(g.psm[m].kind == GENNMI_PSM_EXPCURR) {
                    Isyn += g.psm[m].init * linSyn;
                    linSyn *= g.psm[m].expDecay;
                }
                else {
                    Isyn += linSyn;
                    linSyn = 0.0f;
                }
                if(D) { asGlobal(g.psm[m].denDelay)[((size_t)batch * D + modStep(st.epoch + 1, D)) * n + i] = 0.0f; }
                asGlobal(g.psm[m].outPost)[bi] = linSyn;
            }
        }
        if(numCS) { Isyn += inj[j]; }
        float v0 = l0[j], v1 = l1[j];
        if(g.model == GENNMI_NEURON_LIF) {
            if(v1 <= 0.0f) {
                const float alpha = ((Isyn + g.params[0]) * g.params[1]) + g.params[2];
                v0 = alpha - (g.params[3] * (alpha - v0));
            }
            else {
                v1 -= dt;
            }
            spiked[j] = (v1 <= 0.0f && v0 >= g.params[4]);
            if(spiked[j]) { v0 = g.params[5]; v1 = g.params[6]; }
        }
        else {
            if(v0 >= 30.0f) {
                v0 = g.params[2];
                v1 += g.params[3];
            }
            v0 += 0.5f * (0.04f * v0 * v0 + 5.0f * v0 + 140.0f - v1 + Isyn) * dt;
            v0 += 0.5f * (0.04f * v0 * v0 + 5.0f * v0 + 140.0f - v1 + Isyn) * dt;
            v1 += g.params[0] * (g.params[1] * v0 - v1) * dt;
            if(v0 > 30.0f) { v0 = 30.0f; }
            spiked[j] = (v0 >= 29.99f);
        }
        g.var0[bi] = v0; g.var1[bi] = v1;
    }
    if(localBlock == 0 && batch == 0 && threadIdx.x < g.numPSM) {
        const gennmi_psm_t &psm = g.psm[threadIdx.x];
        if(psm.maxDenDelay && psm.denDelayPtr) { *psm.denDelayPtr = modStep(st.epoch + 1, psm.maxDenDelay); }
    }

    // ---- ordered compaction: rank = spikes of the wave's earlier chunks + spikes of lower lanes in this chunk
    uint32_t rank[NPL];
    uint32_t waveCount = 0;
    #pragma unroll
    for(int j = 0; j < NPL; j++) {
        const uint32_t i = first + j * WAVE;
        const unsigned long long ballot = __ballot(spiked[j]);
        rank[j] = waveCount + __popcll(ballot & ((1ull << lane) - 1ull));
        waveCount += __popcll(ballot);
        if(g.recordSpk && (lane & 31) == 0 && i < n) {
            const uint32_t words = (n + 31) / 32;
            g.recordSpk[((size_t)st.recT * gridDim.y + batch) * words + (i >> 5)] = (uint32_t)(ballot >> (lane & 32));
        }
    }
    if(lane == 0) { shWaveCount[wave] = waveCount; }
    __syncthreads();
    uint32_t blockCount = 0, waveOffset = 0;
    #pragma unroll
    for(uint32_t w = 0; w < BLOCK / WAVE; w++) {
        const uint32_t c = shWaveCount[w];
        if(w < wave) { waveOffset += c; }
        blockCount += c;
    }
    unsigned long long *groupAgg = agg + (size_t)totalNeuronBlocks * gridDim.y;
    const uint32_t prefix = blockQueueOffset(blockCount, localBlock, G.numBlocks, (size_t)batch * totalNeuronBlocks + G.startBlock, agg, groupAgg,
                                             (uint32_t)(st.epoch + 1), &shPrefix, errorFlag);
    if(prefix == 0xFFFFFFFFu) { return; }
    #pragma unroll
    for(int j = 0; j < NPL; j++) {
        if(spiked[j]) { g.spk[(size_t)batch * n + prefix + waveOffset + rank[j]] = first + j * WAVE; }
    }
    if(localBlock == G.numBlocks - 1 && threadIdx.x == 0) { g.spkCnt[batch] = prefix + blockCount; }
}

template<int NPL>
__global__ __launch_bounds__(BLOCK)
void neuronBulkKernel(const NeuronGroupDev * __restrict__ blocks, StepArgs args, float dt, unsigned long long *agg, uint32_t *errorFlag)
{
    neuronBulkBody<NPL>(blocks[blockIdx.x], blockIdx.x, gridDim.x, resolve(args, dt), dt, agg, errorFlag);
}

// One launch per timestep for networks whose projections all go through the dendritic-delay ring: the
// neuron update of step t and the presynaptic update of step t touch disjoint ring slots once zero-delay
// synapses are delivered by the spiking neuron itself, and the presynaptic update reads the shadow spike
// queue of step t-1 while the neuron update refills the visible one.  Neuron blocks come first so that
// their look-back chain starts early.
__global__ __launch_bounds__(BLOCK)
void stepFusedKernel(const NeuronGroupDev * __restrict__ neuronBlocks, uint32_t numNeuronBlocks, const PreGroupDev * __restrict__ preBlocks,
                     StepArgs args, float dt, unsigned long long *agg, uint32_t *errorFlag, unsigned long long *eventCounter)
{
    const Resolved st = resolve(args, dt);
    if(blockIdx.x < numNeuronBlocks) {
        // the neuron blocks are the critical path (other blocks wait for their spike counts): let their
        // instructions issue ahead of the presynaptic blocks that share the compute unit
        __builtin_amdgcn_s_setprio(3);
        neuronBody(neuronBlocks[blockIdx.x], blockIdx.x, numNeuronBlocks, st, dt, agg, errorFlag);
    }
    else { presynapticBody(preBlocks[blockIdx.x - numNeuronBlocks], blockIdx.x - numNeuronBlocks, st, dt, eventCounter); }
}

// Per row: count the synapses with d % D == 0 and, when `entries` is given, append them at offset[row].
__global__ void zeroDelayScanKernel(uint32_t numSrc, uint32_t rowStride, const uint32_t *rowLength, const uint8_t *d, uint32_t D,
                                    const uint32_t *ind, const float *g, float *denDelay, uint32_t numTrg,
                                    uint32_t *zeroLen, const uint32_t *offset, ZeroDelayEntry *entries)
{
    const uint32_t row = blockIdx.x * blockDim.x + threadIdx.x;
    if(row >= numSrc) { return; }
    const size_t base = (size_t)row * rowStride;
    uint32_t count = 0;
    for(uint32_t j = 0; j < rowLength[row]; j++) {
        if((d[base + j] % D) == 0) {
            if(entries) { entries[offset[row] + count] = ZeroDelayEntry{denDelay + ind[base + j], g + base + j, numTrg, D}; }
            count++;
        }
    }
    if(zeroLen) { zeroLen[row] = count; }
}

// Advances the device-resident step state at the end of a captured graph.
// spike sources: (re)build the per-neuron copy of the next spike time from the arrays the user owns
__global__ void nextSpikeTimeKernel(const uint32_t *startSpike, const uint32_t *endSpike, const float *spikeTimes, float *next, size_t count)
{
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if(i < count) {
        const uint32_t s = startSpike[i];
        next[i] = (s != endSpike[i]) ? spikeTimes[s] : INFINITY;
    }
}

__global__ void advanceStepKernel(StepState *state, unsigned long long steps)
{
    if(threadIdx.x == 0 && blockIdx.x == 0) { state->timestep += steps; state->epoch += steps; }
}

// four floats per lane; dwordx4 when both pointers are 16-byte aligned (hipMalloc'd arrays are), else scalar
__global__ void copyKernel(float *dst, const float *src, size_t n)
{
    const size_t i = ((size_t)blockIdx.x * blockDim.x + threadIdx.x) * 4;
    if(i + 4 <= n && ((reinterpret_cast<uintptr_t>(dst) | reinterpret_cast<uintptr_t>(src)) & 15) == 0) {
        *reinterpret_cast<f32x4*>(dst + i) = *reinterpret_cast<const f32x4*>(src + i);
    }
    else {
        for(size_t k = i; k < n && k < i + 4; k++) { dst[k] = src[k]; }
    }
}

__global__ void fillKernel(float *p, float v, size_t n)
{
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if(i < n) { p[i] = v; }
}

// ------------------------------------------------------------------------------------------------
// Remap build: scatter in arbitrary order, then sort every column ascending, which is the order
// the CPU backend's row-major traversal produces (single_threaded_cpu/backend.cc:156-179).
// ------------------------------------------------------------------------------------------------
__global__ void remapCountKernel(uint32_t numSrc, uint32_t rowStride, const uint32_t *rowLength, const uint32_t *ind,
                                 uint32_t colStride, uint32_t *colLength, uint32_t *remap, uint32_t *overflow)
{
    const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t total = (size_t)numSrc * rowStride;
    if(idx >= total) { return; }
    const uint32_t row = (uint32_t)(idx / rowStride), j = (uint32_t)(idx % rowStride);
    if(j >= rowLength[row]) { return; }
    const uint32_t post = ind[idx];
    const uint32_t pos = atomicAdd(&colLength[post], 1u);
    if(remap) {
        if(pos < colStride) { remap[(size_t)post * colStride + pos] = (uint32_t)idx; }
        else { atomicMax(overflow, pos + 1); }
    }
}

__global__ __launch_bounds__(BLOCK)
void remapSortKernel(uint32_t colStride, const uint32_t *colLength, uint32_t *remap)
{
    extern __shared__ uint32_t shCol[];
    const uint32_t col = blockIdx.x;
    const uint32_t len = min(colLength[col], colStride);
    if(len < 2) { return; }
    uint32_t p2 = 1;
    while(p2 < len) { p2 <<= 1; }
    uint32_t *column = remap + (size_t)col * colStride;
    for(uint32_t k = threadIdx.x; k < p2; k += BLOCK) { shCol[k] = (k < len) ? column[k] : 0xFFFFFFFFu; }
    __syncthreads();
    for(uint32_t size = 2; size <= p2; size <<= 1) {
        for(uint32_t stride = size >> 1; stride > 0; stride >>= 1) {
            for(uint32_t k = threadIdx.x; k < p2; k += BLOCK) {
                const uint32_t partner = k ^ stride;
                if(partner > k) {
                    const bool up = ((k & size) == 0);
                    const uint32_t a = shCol[k], b = shCol[partner];
                    if((a > b) == up) { shCol[k] = b; shCol[partner] = a; }
                }
            }
            __syncthreads();
        }
    }
    for(uint32_t k = threadIdx.x; k < len; k += BLOCK) { column[k] = shCol[k]; }
}

uint32_t pow2Floor(uint32_t v) { uint32_t p = 1; while(p * 2 <= v) { p *= 2; } return p; }
uint32_t pow2Ceil(uint32_t v) { uint32_t p = 1; while(p < v) { p *= 2; } return p; }
}   // namespace

// ------------------------------------------------------------------------------------------------
// ------------------------------------------------------------------------------------------------
// Resident plan: many timesteps per launch for networks small enough to live on the chip.
//
// A timestep of such a network moves a few megabytes — half a microsecond of HBM time — but as a chain of
// launches it costs ~12 us: ~4 us per kernel boundary (every L2 is written back and invalidated), then step
// state -> spike count -> spike ids -> rows -> ~10^5 scattered fp32 atomics that retire at ~20 G/s on the memory
// side.  Here one work-group owns RES_T neurons for a whole run: their state stays in registers, their
// postsynaptic input (inSyn) and their slice of every dendritic-delay ring stay in LDS, and the only thing
// work-groups exchange is each step's spikes — one 64-bit word per tile (sequence number, count, and the id
// itself when a single neuron fired; longer lists go through a side buffer).  Every tile reads the words of
// all tiles, looks up which part of each spiking row targets its own neurons (a per-(row, tile) segment table
// built once; rows are sorted by target), and adds those synapses into its LDS ring: no global atomics, no
// global read-modify-write of the ring, no kernel boundary.  The words are double-buffered by step parity: a
// tile can run at most one step ahead of the slowest one, because it needs every tile's word of step s before
// it can publish its own word of step s+1.
//
// The wait for the other tiles' words is bounded (c_spinLimit polls) and also watches the error flag, so a launch
// whose work-groups are not all resident ends with an error instead of hanging.
// ------------------------------------------------------------------------------------------------
constexpr uint32_t RES_T = BLOCK;            // neurons per tile = threads per work-group
constexpr uint32_t RES_MAX_TILES = 1024;
constexpr uint32_t RES_MAX_PROJ = 16;        // projections into one population
constexpr uint32_t RES_MAX_GROUPS = 64;      // neuron groups
constexpr uint32_t RES_PAIR_CAP = 1024;      // (spike, projection) pairs staged per pass
constexpr uint32_t RES_FRONT_MAX = 4;        // front-slot synapses held inline in a segment entry
constexpr uint32_t RES_SEG_OVERFLOW = 1u << 24, RES_SEG_NO_DELAY = 1u << 25;
constexpr uint32_t RES_PAIR_GROUP = 16;      // pairs a wavefront expands at a time
constexpr int RES_SEQ_SHIFT = 41;            // word = seq << 41 | count << 32 | up to four tile-local neuron indices, 8 bits each
constexpr uint32_t RES_WORD_IDS = 4;         // spikes of a tile and step that travel inside its word (more: side buffer)
constexpr uint32_t RES_REPLICAS = 8;         // copies of the word array, one per XCD, so that polling spreads over memory channels

struct ResProj
{
    const uint32_t *ind; const float *g; const uint8_t *d;
    const u32x4 *seg;                   // [numSrc * tilesInGroup][2]: the row's part inside a tile, see residentSegKernel
    uint32_t D;                         // ring depth; 0 = no dendritic delay, events add to inSyn
    uint32_t lds;                       // float offset of the ring (D x RES_T, slot-major) or inSyn row in the tile's LDS
    uint32_t srcGroup, pad_;
};

struct ResTile
{
    uint32_t group, first, count;       // neuron group, first neuron, neurons in this tile
    uint32_t tileInGroup, tilesInGroup, firstTileOfGroup;
    uint32_t numProj, ldsFloats;
    uint32_t ldsIn[GENNMI_MAX_PSM];     // float offset of the inSyn row of postsynaptic model m
    uint32_t ldsRing[GENNMI_MAX_PSM];   // float offset of its ring (when maxDenDelay > 0)
    ResProj proj[RES_MAX_PROJ];
};

// One 32-byte entry per (row, tile of the target population): word 0 = first idSyn of the row's part inside the tile,
// word 1 = its length | number of inline synapses << 16 | flags, words 2-5 = weights and word 6 = the packed tile-local
// targets of up to four synapses whose delay is a multiple of the ring depth.  Those land in the slot the target reads in
// the very step that delivers them, so they are the only ones a step has to wait for; carrying them inside the entry
// saves that step the dependent read of the row.  RES_SEG_OVERFLOW: the segment has more of them than fit (the row part
// is then read at once); RES_SEG_NO_DELAY: the projection has no ring, every synapse is due at once.
__global__ void residentSegKernel(uint32_t numSrc, uint32_t rowStride, const uint32_t *rowLength, const uint32_t *ind, const float *weight,
                                  const uint8_t *delay, uint32_t depth, uint32_t tilesInGroup, u32x4 *seg)
{
    const size_t id = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if(id >= (size_t)numSrc * tilesInGroup) { return; }
    const uint32_t row = (uint32_t)(id / tilesInGroup), tile = (uint32_t)(id % tilesInGroup);
    const uint32_t len = rowLength[row];
    const uint32_t *r = ind + (size_t)row * rowStride;
    auto lowerBound = [&](uint32_t key) {
        uint32_t lo = 0, hi = len;
        while(lo < hi) { const uint32_t mid = (lo + hi) / 2; if(r[mid] < key) { lo = mid + 1; } else { hi = mid; } }
        return lo;
    };
    const uint32_t a = lowerBound(tile * RES_T), b = lowerBound((tile + 1) * RES_T);
    const uint32_t start = row * rowStride + a;
    uint32_t flags = depth ? 0u : RES_SEG_NO_DELAY, numFront = 0, locals = 0;
    uint32_t w[RES_FRONT_MAX] = {0, 0, 0, 0};
    if(depth) {
        for(uint32_t j = a; j < b; j++) {
            if(delay[(size_t)row * rowStride + j] % depth != 0) { continue; }
            if(numFront == RES_FRONT_MAX) { flags |= RES_SEG_OVERFLOW; numFront = 0; break; }    // the row walk adds all of them
            w[numFront] = __float_as_uint(weight[(size_t)row * rowStride + j]);
            locals |= (r[j] - tile * RES_T) << (8 * numFront);
            numFront++;
        }
    }
    u32x4 lo4, hi4;
    lo4.x = start; lo4.y = min(b - a, 0xFFFFu) | (numFront << 16) | flags; lo4.z = w[0]; lo4.w = w[1];
    hi4.x = w[2]; hi4.y = w[3]; hi4.z = locals; hi4.w = 0;
    seg[2 * id] = lo4;
    seg[2 * id + 1] = hi4;
}

// rows must ascend for the segments to be contiguous
__global__ void residentSortedKernel(uint32_t numSrc, uint32_t rowStride, const uint32_t *rowLength, const uint32_t *ind, uint32_t *unsorted)
{
    const size_t id = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if(id >= (size_t)numSrc * rowStride) { return; }
    const uint32_t row = (uint32_t)(id / rowStride), j = (uint32_t)(id % rowStride);
    if(j + 1 < rowLength[row] && ind[id] > ind[id + 1]) { *unsorted = 1; }
}

__device__ __forceinline__ uint32_t waveInclusiveScanU32(uint32_t v, uint32_t lane)
{
    #pragma unroll
    for(int d = 1; d < WAVE; d <<= 1) {
        const uint32_t o = __shfl_up(v, d, WAVE);
        if(lane >= (uint32_t)d) { v += o; }
    }
    return v;
}

__global__ __launch_bounds__(BLOCK)
void residentKernel(const ResTile * __restrict__ tiles, uint32_t numTiles, const NeuronGroupDev * __restrict__ groups,
                    const uint8_t * __restrict__ tileGroup, unsigned long long *tags, uint32_t *side,
                    unsigned long long timestep0, unsigned long long epoch0, unsigned long long numRecordingTimesteps, uint32_t numSteps,
                    float dt, uint32_t zeroDelaySplit, uint32_t *errorFlag, unsigned long long *eventCounter, uint32_t replicaStride)
{
    extern __shared__ float lds[];                       // inSyn rows and ring slices of this tile
    __shared__ unsigned long long shTag[RES_MAX_TILES];
    __shared__ uint2 shPair[RES_PAIR_CAP];               // (presynaptic neuron, projection)
    __shared__ uint2 shSeg[RES_PAIR_CAP];                // (first idSyn, length | flags) of each staged pair
    __shared__ uint32_t shFlagged;                       // staged pairs whose row has to be walked before the update
    __shared__ ResProj shProj[RES_MAX_PROJ];
    __shared__ uint32_t shProjPtr[RES_MAX_PROJ];         // this step's front slot of each projection's ring
    __shared__ uint32_t shProjStart[RES_MAX_GROUPS + 1]; // projections of this tile by source group
    __shared__ uint8_t shProjIdx[RES_MAX_PROJ];
    __shared__ uint8_t shTileGroup[RES_MAX_TILES];
    __shared__ uint32_t shOwn[RES_T];                    // this tile's spikes of the last step, ascending
    __shared__ uint32_t shWave[BLOCK / WAVE];
    __shared__ uint32_t shScalar[4];

    // every tile publishes its word into all copies of the word array and reads the copy of its own XCD
    uint32_t xcc = 0;
    asm volatile("s_getreg_b32 %0, hwreg(HW_REG_XCC_ID)" : "=s"(xcc));
    const unsigned long long *myTags = tags + (size_t)(xcc & (RES_REPLICAS - 1)) * replicaStride;
    const ResTile &T = tiles[blockIdx.x];
    const NeuronGroupDev &G = groups[T.group];
    const gennmi_neuron_update_group_t &g = G.g;
    const uint32_t tid = threadIdx.x, lane = tid & (WAVE - 1), wave = tid / WAVE;
    const uint32_t n = g.numNeurons;
    const uint32_t i = T.first + tid;
    const bool mine = tid < T.count;
    const uint32_t numPSM = g.numPSM, numCS = g.numCS;

    // a launch that finds the error flag raised (an earlier work-group gave up waiting) leaves at once, as one
    if(tid == 0) { shScalar[3] = __hip_atomic_load(errorFlag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
    __syncthreads();
    if(shScalar[3]) { return; }

    // ---- tables into LDS
    for(uint32_t k = tid; k < numTiles; k += BLOCK) { shTileGroup[k] = tileGroup[k]; }
    if(tid < T.numProj) { shProj[tid] = T.proj[tid]; }
    if(tid == 0) {
        // projections grouped by source group (counting sort; a handful of entries)
        for(uint32_t s = 0; s <= RES_MAX_GROUPS; s++) { shProjStart[s] = 0; }
        for(uint32_t p = 0; p < T.numProj; p++) { shProjStart[T.proj[p].srcGroup + 1]++; }
        for(uint32_t s = 0; s < RES_MAX_GROUPS; s++) { shProjStart[s + 1] += shProjStart[s]; }
        for(uint32_t p = 0; p < T.numProj; p++) {
            const uint32_t s = T.proj[p].srcGroup;
            uint32_t before = 0;
            for(uint32_t q = 0; q < p; q++) { before += (T.proj[q].srcGroup == s) ? 1u : 0u; }
            shProjIdx[shProjStart[s] + before] = (uint8_t)p;
        }
    }

    // ---- state: neuron variables in registers, inSyn and ring slices in LDS
    float l0 = 0, l1 = 0;
    if(mine) { l0 = asGlobal(g.var0)[i]; l1 = asGlobal(g.var1)[i]; }
    for(uint32_t m = 0; m < numPSM; m++) {
        lds[T.ldsIn[m] + tid] = mine ? asGlobal(g.psm[m].outPost)[i] : 0.0f;
        const uint32_t D = g.psm[m].maxDenDelay;
        for(uint32_t slot = 0; slot < D; slot++) {
            lds[T.ldsRing[m] + slot * RES_T + tid] = mine ? asGlobal(g.psm[m].denDelay)[(size_t)slot * n + i] : 0.0f;
        }
    }

    // ---- this tile's spikes of the step before the first one, from the population's (ascending) queue
    if(tid == 0) { shScalar[0] = 0; shScalar[1] = 0; }
    __syncthreads();
    {
        const uint32_t cnt = asGlobal(g.spkCnt)[0];
        uint32_t below = 0, inside = 0;
        for(uint32_t k = tid; k < cnt; k += BLOCK) {
            const uint32_t id = asGlobal(g.spk)[k];
            below += (id < T.first) ? 1u : 0u;
            inside += (id >= T.first && id < T.first + T.count) ? 1u : 0u;
        }
        if(below) { atomicAdd(&shScalar[0], below); }
        if(inside) { atomicAdd(&shScalar[1], inside); }
        __syncthreads();
        const uint32_t lo = shScalar[0];
        for(uint32_t k = tid; k < cnt; k += BLOCK) {
            const uint32_t id = asGlobal(g.spk)[k];
            if(id >= T.first && id < T.first + T.count) { shOwn[k - lo] = id; }
        }
    }
    __syncthreads();
    uint32_t ownCount = shScalar[1];

    // (callers synchronise the work-group after filling shOwn)
    auto publish = [&](uint32_t seq, uint32_t count) {
        const uint32_t parity = seq & 1u;
        if(count > RES_WORD_IDS) {
            for(uint32_t r = tid; r < count; r += BLOCK) {
                __hip_atomic_store(&side[((size_t)parity * numTiles + blockIdx.x) * RES_T + r], shOwn[r], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
            // the ids must have reached memory before the word that announces them
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "agent");
            __syncthreads();
        }
        if(tid < RES_REPLICAS) {
            uint32_t locals = 0;
            for(uint32_t e = 0; e < min(count, RES_WORD_IDS); e++) { locals |= (shOwn[e] - T.first) << (8 * e); }
            const unsigned long long word = ((unsigned long long)seq << RES_SEQ_SHIFT) | ((unsigned long long)count << 32) | locals;
            __hip_atomic_store(&tags[(size_t)tid * replicaStride + (size_t)parity * numTiles + blockIdx.x], word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    };

    // source tiles this thread watches (tile tid, tid + 256, ...) and how many of this tile's projections each feeds
    constexpr uint32_t WATCH = RES_MAX_TILES / BLOCK;
    uint32_t watchProj0[WATCH], watchNumProj[WATCH], watchFirst[WATCH];
    #pragma unroll
    for(uint32_t q = 0; q < WATCH; q++) {
        const uint32_t k = tid + q * BLOCK;
        watchFirst[q] = (k < numTiles) ? tiles[k].first : 0u;
        const uint32_t s = (k < numTiles) ? shTileGroup[k] : 0u;
        watchProj0[q] = shProjStart[s];
        watchNumProj[q] = (k < numTiles) ? shProjStart[s + 1] - shProjStart[s] : 0u;
    }

    // Waits for every tile's word of sequence number seq (false when the bounded wait expired somewhere) and stages the
    // (spike, projection) pairs that concern this tile in shPair; shScalar[0] receives their number, which may exceed
    // RES_PAIR_CAP (then only the claims that fitted were written and the caller takes the chunked path).
    auto poll = [&](uint32_t seq, unsigned long long epoch) -> bool {
        const uint32_t parity = seq & 1u;
        bool ok = true;
        unsigned long long word[WATCH];
        uint32_t pending = 0;
        #pragma unroll
        for(uint32_t q = 0; q < WATCH; q++) { word[q] = 0; if(tid + q * BLOCK < numTiles) { pending |= 1u << q; } }
        if(tid == 0) { shScalar[0] = 0; shFlagged = 0; }
        uint32_t spins = 0;
        while(pending) {
            #pragma unroll
            for(uint32_t q = 0; q < WATCH; q++) {
                if(pending & (1u << q)) {
                    word[q] = __hip_atomic_load(&myTags[(size_t)parity * numTiles + tid + q * BLOCK], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                }
            }
            #pragma unroll
            for(uint32_t q = 0; q < WATCH; q++) {
                if((pending & (1u << q)) && (uint32_t)(word[q] >> RES_SEQ_SHIFT) == seq) { pending &= ~(1u << q); }
            }
            if(!pending) { break; }
            ++spins;
            if(spins > c_spinLimit || ((spins & 255u) == 0 && __hip_atomic_load(errorFlag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT))) { ok = false; break; }
            __builtin_amdgcn_s_sleep(1);
        }
        #pragma unroll
        for(uint32_t q = 0; q < WATCH; q++) { if(tid + q * BLOCK < numTiles) { shTag[tid + q * BLOCK] = word[q]; } }
        const bool allOk = __syncthreads_and(ok ? 1 : 0) != 0;
        if(!allOk) {
            if(tid == 0) { atomicOr(errorFlag, 1u); }
            return false;
        }
        // front slot of every projection's ring in the step this exchange feeds
        if(tid < T.numProj) { shProjPtr[tid] = shProj[tid].D ? modStep(epoch + 1, shProj[tid].D) : 0u; }
        #pragma unroll
        for(uint32_t q = 0; q < WATCH; q++) {
            const uint32_t c = (uint32_t)(word[q] >> 32) & 0x1FFu, np = watchNumProj[q];
            if(c == 0 || np == 0) { continue; }
            uint32_t pos = atomicAdd(&shScalar[0], c * np);
            if(pos + c * np > RES_PAIR_CAP) { continue; }
            for(uint32_t e = 0; e < c; e++) {
                const uint32_t id = (c <= RES_WORD_IDS) ? watchFirst[q] + (((uint32_t)word[q] >> (8 * e)) & 0xFFu)
                                                        : __hip_atomic_load(&side[((size_t)parity * numTiles + tid + q * BLOCK) * RES_T + e], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                for(uint32_t j = 0; j < np; j++) { shPair[pos++] = make_uint2(id, shProjIdx[watchProj0[q] + j]); }
            }
        }
        __syncthreads();
        return true;
    };

    unsigned long long events = 0;

    constexpr uint32_t PASS_ALL = 0, PASS_LATER = 1, PASS_DUE = 2;      // which synapses a pass adds: see process()

    // First pass over the staged pairs, one lane per pair: reads the pair's segment entry, keeps (start, length, flags)
    // for the passes that walk the row, and — unless `skipInline` — adds the entry's inline synapses to the front slot.
    auto readSegments = [&](uint32_t numPairs, bool skipInline, bool count) {
        for(uint32_t q = tid; q < numPairs; q += BLOCK) {
            const uint2 pr = shPair[q];
            const ResProj &P = shProj[pr.y];
            GLOBAL_AS const u32x4 *entry = asGlobal(P.seg) + 2 * ((size_t)pr.x * T.tilesInGroup + T.tileInGroup);
            const u32x4 lo4 = entry[0], hi4 = entry[1];
            shSeg[q] = make_uint2(lo4.x, lo4.y);
            if(lo4.y & (RES_SEG_OVERFLOW | RES_SEG_NO_DELAY)) { atomicAdd(&shFlagged, 1u); }
            if(count) { events += lo4.y & 0xFFFFu; }
            if(skipInline) { continue; }
            const uint32_t numFront = (lo4.y >> 16) & 0xFFu;
            const uint32_t frontBase = P.lds + shProjPtr[pr.y] * RES_T;
            const uint32_t w[RES_FRONT_MAX] = {lo4.z, lo4.w, hi4.x, hi4.y};
            #pragma unroll
            for(uint32_t f = 0; f < RES_FRONT_MAX; f++) {
                if(f < numFront) { unsafeAtomicAdd(&lds[frontBase + ((hi4.z >> (8 * f)) & 0xFFu)], __uint_as_float(w[f])); }
            }
        }
    };

    // Walks the row segments of the staged pairs, 16 pairs per wavefront at a time, all lanes sharing their synapses.
    // A synapse is "due" when it lands in the slot read this step (delay a multiple of the ring depth, or no ring).
    // PASS_ALL adds every synapse, PASS_LATER those not due, PASS_DUE the due ones; `flaggedOnly` restricts the walk to
    // segments whose due synapses are not all inline in their entry.
    auto process = [&](uint32_t numPairs, uint32_t pass, bool flaggedOnly) {
        for(uint32_t q0 = wave * RES_PAIR_GROUP; q0 < numPairs; q0 += (BLOCK / WAVE) * RES_PAIR_GROUP) {
            uint32_t len = 0, start = 0, proj = 0;
            if(lane < RES_PAIR_GROUP && q0 + lane < numPairs) {
                const uint2 sg = shSeg[q0 + lane];
                proj = shPair[q0 + lane].y;
                const bool flagged = (sg.y & (RES_SEG_OVERFLOW | RES_SEG_NO_DELAY)) != 0;
                const bool skip = (flaggedOnly && !flagged) || (pass == PASS_LATER && (sg.y & RES_SEG_NO_DELAY));
                start = sg.x; len = skip ? 0u : (sg.y & 0xFFFFu);
            }
            const uint32_t incl = waveInclusiveScanU32(len, lane);
            const uint32_t sum = __shfl(incl, WAVE - 1, WAVE);
            for(uint32_t f0 = 0; f0 < sum; f0 += 4 * WAVE) {
                uint32_t post[4], slotPtr[4], ldsBase[4], depth[4], dly[4]; float w[4]; bool valid[4];
                #pragma unroll
                for(int u = 0; u < 4; u++) {
                    const uint32_t f = f0 + u * WAVE + lane;
                    valid[u] = f < sum;
                    uint32_t j = 0;
                    #pragma unroll
                    for(uint32_t step = RES_PAIR_GROUP / 2; step > 0; step >>= 1) {
                        const uint32_t v = __shfl(incl, j + step - 1, WAVE);
                        if(v <= f) { j += step; }
                    }
                    const uint32_t lenJ = __shfl(len, j, WAVE), startJ = __shfl(start, j, WAVE), projJ = __shfl(proj, j, WAVE);
                    const uint32_t inclJ = __shfl(incl, j, WAVE);
                    post[u] = 0; w[u] = 0.0f; dly[u] = 0; depth[u] = 0; ldsBase[u] = 0; slotPtr[u] = 0;
                    if(valid[u]) {
                        const ResProj &P = shProj[projJ];
                        const uint32_t syn = startJ + (f - (inclJ - lenJ));
                        post[u] = asGlobal(P.ind)[syn];
                        w[u] = asGlobal(P.g)[syn];
                        depth[u] = P.D; ldsBase[u] = P.lds; slotPtr[u] = shProjPtr[projJ];
                        if(P.D) { dly[u] = asGlobal(P.d)[syn]; }
                    }
                }
                #pragma unroll
                for(int u = 0; u < 4; u++) {
                    const uint32_t local = post[u] - T.first;
                    if(!valid[u] || local >= RES_T) { continue; }
                    const uint32_t slot = depth[u] ? (slotPtr[u] + dly[u]) % depth[u] : 0u;
                    const bool due = !depth[u] || (slot == slotPtr[u]);
                    if((pass == PASS_LATER && due) || (pass == PASS_DUE && !due)) { continue; }
                    unsafeAtomicAdd(&lds[ldsBase[u] + slot * RES_T + local], w[u]);
                }
            }
        }
    };

    // the pairs of a step that holds more of them than shPair does: staged and walked RES_PAIR_CAP at a time, in full
    auto processChunked = [&](uint32_t seq, uint32_t total, uint32_t pass, bool count) {
        const uint32_t parity = seq & 1u;
        uint32_t want = 0;
        for(uint32_t k = tid; k < numTiles; k += BLOCK) {
            const uint32_t c = (uint32_t)(shTag[k] >> 32) & 0x1FFu;
            const uint32_t s = shTileGroup[k];
            want += c * (shProjStart[s + 1] - shProjStart[s]);
        }
        const uint32_t inclusive = waveInclusiveScanU32(want, lane);
        if(lane == WAVE - 1) { shWave[wave] = inclusive; }
        __syncthreads();
        uint32_t base = inclusive - want;
        #pragma unroll
        for(uint32_t w = 0; w < BLOCK / WAVE; w++) { if(w < wave) { base += shWave[w]; } }
        for(uint32_t chunk0 = 0; chunk0 < total; chunk0 += RES_PAIR_CAP) {
            uint32_t pos = base;
            for(uint32_t k = tid; k < numTiles; k += BLOCK) {
                const unsigned long long tag = shTag[k];
                const uint32_t c = (uint32_t)(tag >> 32) & 0x1FFu;
                const uint32_t s = shTileGroup[k];
                const uint32_t p0 = shProjStart[s], np = shProjStart[s + 1] - p0;
                if(c == 0 || np == 0) { continue; }
                if(pos + c * np <= chunk0 || pos >= chunk0 + RES_PAIR_CAP) { pos += c * np; continue; }
                for(uint32_t q = 0; q < c; q++) {
                    const uint32_t id = (c <= RES_WORD_IDS) ? tiles[k].first + (((uint32_t)tag >> (8 * q)) & 0xFFu)
                                                            : __hip_atomic_load(&side[((size_t)parity * numTiles + k) * RES_T + q], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    for(uint32_t j = 0; j < np; j++, pos++) {
                        if(pos >= chunk0 && pos < chunk0 + RES_PAIR_CAP) { shPair[pos - chunk0] = make_uint2(id, shProjIdx[p0 + j]); }
                    }
                }
            }
            __syncthreads();
            const uint32_t numPairs = min(RES_PAIR_CAP, total - chunk0);
            readSegments(numPairs, true, count);
            __syncthreads();
            process(numPairs, pass, false);
            __syncthreads();
        }
    };

    // After a successful poll(seq): what the spikes of that exchange owe this tile NOW — the synapses due this step
    // (inline in the segment entries; row walks only for segments that say so).  `convention` is PASS_ALL normally,
    // PASS_LATER when a previous launch has already delivered the due synapses of these spikes, PASS_DUE when only those
    // are wanted.  Returns the number of staged pairs whose remaining synapses deliverLater() has to add, or 0.
    auto deliverDue = [&](uint32_t seq, uint32_t convention) -> uint32_t {
        const uint32_t total = shScalar[0];
        if(total > RES_PAIR_CAP) {
            processChunked(seq, total, convention, convention != PASS_DUE);
            return 0u;
        }
        readSegments(total, convention == PASS_LATER, convention != PASS_DUE);
        __syncthreads();
        if(convention != PASS_LATER && shFlagged) { process(total, PASS_DUE, true); }
        return (convention == PASS_DUE) ? 0u : total;
    };
    // the rest of those pairs' synapses: none of them is read before the next step
    auto deliverLater = [&](uint32_t numPairs) {
        if(numPairs) { process(numPairs, PASS_LATER, false); }
    };

    // ---- exchange the spikes that precede the first step, then step
    publish(1u, ownCount);
    bool ok = true;
    uint32_t k = 0;
    for(; k < numSteps; k++) {
        const unsigned long long epoch = epoch0 + k;
        if(!poll(k + 1, epoch)) { ok = false; break; }
        const uint32_t later = deliverDue(k + 1, (zeroDelaySplit && k == 0) ? PASS_LATER : PASS_ALL);
        __syncthreads();

        // neuron update: same operations in the same order as neuronBody
        bool spiked = false;
        if(mine) {
            float Isyn = 0;
            #pragma unroll
            for(uint32_t m = 0; m < GENNMI_MAX_PSM; m++) {
                if(m < numPSM) {
                    float linSyn = lds[T.ldsIn[m] + tid];
                    const uint32_t D = g.psm[m].maxDenDelay;
                    if(D) {
                        const uint32_t front = T.ldsRing[m] + modStep(epoch + 1, D) * RES_T + tid;
                        linSyn += lds[front];
                        lds[front] = 0.0f;
                    }
                    if(g.psm[m].kind == GENNMI_PSM_EXPCURR) {
                        Isyn += g.psm[m].init * linSyn;
                        linSyn *= g.psm[m].expDecay;
                    }
                    else {
                        Isyn += linSyn;
                        linSyn = 0.0f;
                    }
                    lds[T.ldsIn[m] + tid] = linSyn;
                }
            }
            #pragma unroll
            for(uint32_t c = 0; c < GENNMI_MAX_CS; c++) { if(c < numCS) { Isyn += g.cs[c].amp; } }
            if(g.model == GENNMI_NEURON_LIF) {
                if(l1 <= 0.0f) {
                    const float alpha = ((Isyn + g.params[0]) * g.params[1]) + g.params[2];
                    l0 = alpha - (g.params[3] * (alpha - l0));
                }
                else {
                    l1 -= dt;
                }
                spiked = (l1 <= 0.0f && l0 >= g.params[4]);
                if(spiked) { l0 = g.params[5]; l1 = g.params[6]; }
            }
            else {
                if(l0 >= 30.0f) {
                    l0 = g.params[2];
                    l1 += g.params[3];
                }
                l0 += 0.5f * (0.04f * l0 * l0 + 5.0f * l0 + 140.0f - l1 + Isyn) * dt;
                l0 += 0.5f * (0.04f * l0 * l0 + 5.0f * l0 + 140.0f - l1 + Isyn) * dt;
                l1 += g.params[0] * (g.params[1] * l0 - l1) * dt;
                if(l0 > 30.0f) { l0 = 30.0f; }
                spiked = (l0 >= 29.99f);
            }
        }
        const unsigned long long ballot = __ballot(spiked);
        const uint32_t laneRank = __popcll(ballot & ((1ull << lane) - 1ull));
        if(lane == 0) { shWave[wave] = __popcll(ballot); }
        if(g.recordSpk && (lane & 31) == 0 && mine) {
            const unsigned long long ts = timestep0 + k;
            const uint32_t recT = numRecordingTimesteps ? (((ts | numRecordingTimesteps) >> 32) ? (uint32_t)(ts % numRecordingTimesteps)
                                                                                                : ((uint32_t)ts % (uint32_t)numRecordingTimesteps)) : 0u;
            g.recordSpk[(size_t)recT * ((n + 31) / 32) + (i >> 5)] = (uint32_t)(ballot >> (lane & 32));
        }
        __syncthreads();
        uint32_t waveOffset = 0;
        ownCount = 0;
        #pragma unroll
        for(uint32_t w = 0; w < BLOCK / WAVE; w++) {
            const uint32_t c = shWave[w];
            if(w < wave) { waveOffset += c; }
            ownCount += c;
        }
        if(spiked) { shOwn[waveOffset + laneRank] = i; }
        __syncthreads();
        publish(k + 2, ownCount);
        // while the words of this step travel: the synapses of the previous step's spikes that are not due yet
        deliverLater(later);
    }

    // ---- after the last step: everybody's last spikes give the position of this tile's spikes in the population's
    // queue; a runner that delivers front-slot synapses one step early (single-launch plan) wants them in the ring now
    const unsigned long long epochEnd = epoch0 + numSteps;       // completed steps
    if(ok && !poll(numSteps + 1, epochEnd)) { ok = false; }
    if(!ok) { return; }
    if(zeroDelaySplit) { deliverDue(numSteps + 1, PASS_DUE); }
    __syncthreads();

    if(mine) { asGlobal(g.var0)[i] = l0; asGlobal(g.var1)[i] = l1; }
    for(uint32_t m = 0; m < numPSM; m++) {
        if(mine) { asGlobal(g.psm[m].outPost)[i] = lds[T.ldsIn[m] + tid]; }
        const uint32_t D = g.psm[m].maxDenDelay;
        for(uint32_t slot = 0; slot < D; slot++) {
            if(mine) { asGlobal(g.psm[m].denDelay)[(size_t)slot * n + i] = lds[T.ldsRing[m] + slot * RES_T + tid]; }
        }
        if(T.tileInGroup == 0 && tid == 0 && D && g.psm[m].denDelayPtr) { *g.psm[m].denDelayPtr = modStep(epochEnd, D); }
    }
    uint32_t offset = 0;
    for(uint32_t q = T.firstTileOfGroup + tid; q < T.firstTileOfGroup + T.tileInGroup; q += BLOCK) { offset += (uint32_t)(shTag[q] >> 32) & 0x1FFu; }
    if(tid == 0) { shScalar[2] = 0; }
    __syncthreads();
    if(offset) { atomicAdd(&shScalar[2], offset); }
    __syncthreads();
    offset = shScalar[2];
    const bool lastTile = (T.tileInGroup == T.tilesInGroup - 1);
    const uint32_t shadowParity = (uint32_t)((epochEnd - 1) & 1);
    for(uint32_t r = tid; r < ownCount; r += BLOCK) {
        const uint32_t id = shOwn[r];
        g.spk[offset + r] = id;
        for(uint32_t q = 0; q < g.numExtraSpk; q++) { g.extraSpk[q][offset + r] = id; }
        if(G.shadowSpk) { G.shadowSpk[(size_t)shadowParity * n + offset + r] = id; }
    }
    if(lastTile && tid == 0) {
        g.spkCnt[0] = offset + ownCount;
        for(uint32_t q = 0; q < g.numExtraSpk; q++) { g.extraSpkCnt[q][0] = offset + ownCount; }
        if(G.shadowSpk) { G.shadowCnt[shadowParity] = offset + ownCount; }
    }
    for(int off = WAVE / 2; off > 0; off >>= 1) { events += __shfl_down(events, off, WAVE); }
    if(lane == 0 && events) { atomicAdd(eventCounter, events); }
}

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
    StepState *dState = nullptr;
    unsigned long long epoch = 0;       // completed steps (host mirror)
    bool synapsesDone = false;          // updateSynapses ran for the current step
    bool fusedStep = false;             // zero-delay synapses are delivered by the neuron update; one launch per step
    TileGroupDev *dTile = nullptr; uint32_t tileBlocks = 0, tileFloats = 0, tileThreads = BLOCK;
    uint32_t postLdsBytes = 0;
    ConvTileDev *dConvTile = nullptr; uint32_t convTileBlocks = 0; size_t convTileBytes = 0;
    std::vector<void*> owned;           // engine-private device allocations (shadow queues, zero-delay lists)
    // resident plan (many steps per launch)
    bool resident = false;
    ResTile *dResTiles = nullptr; NeuronGroupDev *dResGroups = nullptr; uint8_t *dResTileGroup = nullptr;
    unsigned long long *dResTags = nullptr; uint32_t *dResSide = nullptr;
    uint32_t resTiles = 0, resReplicaStride = 0; size_t resLdsBytes = 0;
    std::vector<u32x4*> resSegs;        // segment table of each presynaptic group, in push order
    std::vector<uint32_t> resSegTiles;  // tiles of its target population
    uint32_t neuronsPerLane = 1;        // 2, 4 or 8: neuronBulkKernel instead of neuronUpdateKernel
    bool sourcesStale = false;          // startSpike / endSpike / spikeTimes of a spike source were written since nextSpikeTime was built
    bool resStale = false;              // connectivity or weights were written since the tables were built
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
            if(n.g.model != GENNMI_NEURON_SPIKE_SOURCE_ARRAY || r->sourcesStale) { continue; }
            const size_t perNeuron = (size_t)r->batch * n.g.numNeurons * sizeof(uint32_t);
            const uintptr_t st = reinterpret_cast<uintptr_t>(n.g.startSpike), en = reinterpret_cast<uintptr_t>(n.g.endSpike);
            if((a < st + perNeuron && st < b) || (a < en + perNeuron && en < b) || (a < reinterpret_cast<uintptr_t>(n.g.spikeTimes) + n.spikeTimesBytes && reinterpret_cast<uintptr_t>(n.g.spikeTimes) < b)) { r->sourcesStale = true; }
        }
        if(!r->resident || r->resStale) { continue; }
        for(const auto &p : r->pre) {
            const size_t entries = (size_t)p.g.numSrcNeurons * p.g.rowStride;
            const struct { const void *ptr; size_t size; } arrays[] = {
                {p.g.g, entries * sizeof(float)}, {p.g.ind, entries * sizeof(uint32_t)}, {p.g.d, p.g.d ? entries : 0},
                {p.g.rowLength, (size_t)p.g.numSrcNeurons * sizeof(uint32_t)}};
            for(const auto &arr : arrays) {
                const uintptr_t lo = reinterpret_cast<uintptr_t>(arr.ptr);
                if(arr.size && a < lo + arr.size && lo < b) { r->resStale = true; }
            }
        }
    }
}

namespace gennmi_detail
{
// error reporting and write tracking for the library's other translation units
int fail(int code, const std::string &msg) { return ::fail(code, msg); }
void noteDeviceWrite(const void *dev, size_t bytes) { ::noteDeviceWrite(dev, bytes); }
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
    return GENNMI_OK;
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
int gennmi_free(void *devPtr) { HIP_TRY(hipFree(devPtr)); return GENNMI_OK; }
int gennmi_memcpy_to_device(void *dev, const void *host, size_t bytes)
{
    HIP_TRY(hipMemcpy(dev, host, bytes, hipMemcpyHostToDevice));
    noteDeviceWrite(dev, bytes);
    return GENNMI_OK;
}
int gennmi_memcpy_from_device(void *host, const void *dev, size_t bytes) { HIP_TRY(hipMemcpy(host, dev, bytes, hipMemcpyDeviceToHost)); return GENNMI_OK; }
int gennmi_memset(void *dev, int value, size_t bytes)
{
    HIP_TRY(hipMemset(dev, value, bytes));
    noteDeviceWrite(dev, bytes);
    return GENNMI_OK;
}
int gennmi_fill_f32(float *dev, float value, size_t count)
{
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
int gennmi_synchronize(void) { HIP_TRY(hipDeviceSynchronize()); return GENNMI_OK; }

// ---- host mirrors: host buffer <-> device buffer pairs, for callers whose generated code only knows host pointers
namespace
{
struct Mirror { void *dev; size_t bytes; };
std::map<uintptr_t, Mirror> g_mirrors;      // keyed by host base address
std::mutex g_mirrorMutex;
}
int gennmi_register_mirror(const void *host, void *dev, size_t bytes)
{
    if(!host || !dev || bytes == 0) { return fail(GENNMI_EINVAL, "register_mirror: null pointer or empty buffer"); }
    std::lock_guard<std::mutex> lock(g_mirrorMutex);
    g_mirrors[reinterpret_cast<uintptr_t>(host)] = Mirror{dev, bytes};
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
int gennmi_push_mirrors(void)
{
    std::lock_guard<std::mutex> lock(g_mirrorMutex);
    for(const auto &m : g_mirrors) {
        HIP_TRY(hipMemcpy(m.second.dev, reinterpret_cast<const void*>(m.first), m.second.bytes, hipMemcpyHostToDevice));
        noteDeviceWrite(m.second.dev, m.second.bytes);
    }
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
    HIP_TRY(hipMalloc(&r->dError, sizeof(uint32_t)));
    HIP_TRY(hipMemset(r->dError, 0, sizeof(uint32_t)));
    HIP_TRY(hipMalloc(&r->dEvents, sizeof(unsigned long long)));
    HIP_TRY(hipMemset(r->dEvents, 0, sizeof(unsigned long long)));
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
    {
        std::lock_guard<std::mutex> lock(g_runnersMutex);
        g_runners.erase(std::remove(g_runners.begin(), g_runners.end(), r), g_runners.end());
    }
    hipStreamSynchronize(r->stream);
    if(r->graphExec) { hipGraphExecDestroy(r->graphExec); }
    for(hipEvent_t e : r->eventPool) { hipEventDestroy(e); }
    for(hipEvent_t e : r->marks) { if(e) { hipEventDestroy(e); } }
    for(void *q : r->owned) { hipFree(q); }
    hipFree(r->dTile); hipFree(r->dConvTile);
    hipFree(r->dNeuron); hipFree(r->dPre); hipFree(r->dPost); hipFree(r->dDense); hipFree(r->dProc); hipFree(r->dAgg); hipFree(r->dError); hipFree(r->dEvents); hipFree(r->dState);
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
        if(g->cs[c].kind > GENNMI_CS_ARRAY) { return fail(GENNMI_EUNSUPPORTED, "push_neuron_update_group: unknown current source"); }
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
        if(g->wum == GENNMI_WUM_STDP_TRACE) { return fail(GENNMI_EUNSUPPORTED, "push_presynaptic_update_group: axonal delay on a plastic projection"); }
    }
    else if(g->axonalDelaySteps) { return fail(GENNMI_EINVAL, "push_presynaptic_update_group: axonal delay without delay slots"); }
    PreGroupDev d;
    memset(&d, 0, sizeof(d));
    d.g = *g;
    if(g->matrix == GENNMI_MATRIX_SPARSE) {
        if(!g->rowLength || !g->ind || g->rowStride == 0) { return fail(GENNMI_EINVAL, "push_presynaptic_update_group: sparse arrays missing"); }
        if((uint64_t)g->numSrcNeurons * g->rowStride > 0xFFFFFFFFull) { return fail(GENNMI_EUNSUPPORTED, "push_presynaptic_update_group: synapse index exceeds 32 bits"); }
        if(g->wum == GENNMI_WUM_STATIC_PULSE_DENDRITIC_DELAY) {
            if(!g->d || !g->denDelay || g->maxDenDelay == 0) { return fail(GENNMI_EINVAL, "push_presynaptic_update_group: dendritic delay arrays missing"); }
        }
        else if(g->wum == GENNMI_WUM_STDP_TRACE) {
            if(!g->trgST || !g->postTrace) { return fail(GENNMI_EINVAL, "push_presynaptic_update_group: STDP arrays missing"); }
            if(r->batch != 1) { return fail(GENNMI_EUNSUPPORTED, "push_presynaptic_update_group: plastic weights need batch size 1"); }
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
    if(!g->colLength || !g->remap || !g->g || !g->trgSpk || !g->trgSpkCnt || !g->srcST || !g->preTrace) {
        return fail(GENNMI_EINVAL, "push_postsynaptic_update_group: required array missing");
    }
    if(g->rowStride == 0 || g->colStride == 0) { return fail(GENNMI_EINVAL, "push_postsynaptic_update_group: zero stride"); }
    if(r->batch != 1) { return fail(GENNMI_EUNSUPPORTED, "push_postsynaptic_update_group: plastic weights need batch size 1"); }
    if((g->rowLength == nullptr) != (g->ind == nullptr)) { return fail(GENNMI_EINVAL, "push_postsynaptic_update_group: rowLength and ind go together"); }
    PostGroupDev d;
    memset(&d, 0, sizeof(d));
    d.g = *g;
    if(idx) { *idx = (uint32_t)r->post.size(); }
    r->post.push_back(d);
    return GENNMI_OK;
}

// Resident plan (residentKernel): chosen when the whole network fits the chip — batch 1, static SPARSE projections
// (with or without dendritic delay) with ascending rows between LIF / Izhikevich populations driven by DC sources, every
// tile of 256 neurons with its ring slices in LDS and all tiles resident at once.  GENNMI_RESIDENT=0 disables it.
static int setupResident(gennmi_runner *r, uint32_t numCU)
{
    const char *env = getenv("GENNMI_RESIDENT");
    if(env && atoi(env) == 0) { return GENNMI_OK; }
    if(r->batch != 1 || !r->post.empty() || r->pre.empty() || !r->dense.empty() || !r->proc.empty() || r->neuron.size() > RES_MAX_GROUPS) { return GENNMI_OK; }
    for(const auto &n : r->neuron) {
        const auto &g = n.g;
        if((g.model != GENNMI_NEURON_LIF && g.model != GENNMI_NEURON_IZHIKEVICH) || g.preTrace || g.postTrace || g.sT || g.numDelaySlots > 1 || g.numSpkEvent || g.numPreOutput) { return GENNMI_OK; }
        for(uint32_t c = 0; c < g.numCS; c++) { if(g.cs[c].kind != GENNMI_CS_DC) { return GENNMI_OK; } }
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
    if(ldsBytes > 32 * 1024) {
        HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void*>(residentKernel), hipFuncAttributeMaxDynamicSharedMemorySize, (int)ldsBytes));
    }
    int perCU = 0;
    HIP_TRY(hipOccupancyMaxActiveBlocksPerMultiprocessor(&perCU, residentKernel, BLOCK, ldsBytes));
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
        ResProj proj{};
        proj.ind = q.ind; proj.g = q.g; proj.d = q.d; proj.seg = dSeg;
        proj.D = (q.wum == GENNMI_WUM_STATIC_PULSE_DENDRITIC_DELAY) ? q.maxDenDelay : 0u;
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
    HIP_TRY(hipMalloc(&r->dResSide, 2 * tiles.size() * RES_T * sizeof(uint32_t)));
    r->owned.push_back(r->dResSide);
    r->resTiles = (uint32_t)tiles.size();
    r->resLdsBytes = ldsBytes;
    r->resident = true;
    return GENNMI_OK;
}

// `numSteps` steps of a network on the resident plan, as few launches as the sequence counter allows
static int launchResident(gennmi_runner *r, unsigned long long timestep, unsigned long long numSteps, unsigned long long numRecordingTimesteps)
{
    constexpr unsigned long long MAX_STEPS = 1ull << 20;
    bool stale;
    {
        std::lock_guard<std::mutex> lock(g_runnersMutex);
        stale = r->resStale;
        r->resStale = false;
    }
    if(stale) {
        // weights or connectivity were written since the segment tables were built: the inline synapses may be out of date
        for(size_t k = 0; k < r->pre.size(); k++) {
            const auto &q = r->pre[k].g;
            const size_t entries = (size_t)q.numSrcNeurons * r->resSegTiles[k];
            const uint32_t depth = (q.wum == GENNMI_WUM_STATIC_PULSE_DENDRITIC_DELAY) ? q.maxDenDelay : 0u;
            residentSegKernel<<<dim3((unsigned int)((entries + BLOCK - 1) / BLOCK)), dim3(BLOCK), 0, r->stream>>>(
                q.numSrcNeurons, q.rowStride, q.rowLength, q.ind, q.g, q.d, depth, r->resSegTiles[k], r->resSegs[k]);
        }
        HIP_TRY(hipGetLastError());
    }
    for(unsigned long long done = 0; done < numSteps; ) {
        const uint32_t chunk = (uint32_t)std::min(MAX_STEPS, numSteps - done);
        HIP_TRY(hipMemsetAsync(r->dResTags, 0, (size_t)RES_REPLICAS * r->resReplicaStride * sizeof(unsigned long long), r->stream));
        residentKernel<<<dim3(r->resTiles), dim3(BLOCK), r->resLdsBytes, r->stream>>>(
            r->dResTiles, r->resTiles, r->dResGroups, r->dResTileGroup, r->dResTags, r->dResSide, timestep + done, r->epoch, numRecordingTimesteps,
            chunk, r->dt, r->fusedStep ? 1u : 0u, r->dError, r->dEvents, r->resReplicaStride);
        HIP_TRY(hipGetLastError());
        done += chunk;
        r->epoch += chunk;
    }
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

    // a projection's view of its source's delay slots must be the source's own
    for(const auto &p : r->pre) {
        for(const auto &n : r->neuron) {
            if(n.g.spk == p.g.srcSpk && std::max(1u, n.g.numDelaySlots) != std::max(1u, p.g.numSrcDelaySlots)) {
                return fail(GENNMI_EINVAL, "runner_finalise: a projection and its source population disagree on the number of delay slots");
            }
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
    }
    const uint32_t neuronsPerBlock = BLOCK * r->neuronsPerLane;
    uint32_t block = 0;
    for(auto &n : r->neuron) {
        n.startBlock = block;
        n.numBlocks = (n.g.numNeurons + neuronsPerBlock - 1) / neuronsPerBlock;
        block += n.numBlocks;
    }
    r->neuronBlocks = block;

    // Presynaptic launch geometry.  The number of spikes is only known on the device, so every
    // group gets a fixed number of blocks and deals its (spike, chunk) work items round-robin to their
    // sub-groups.  A group wants enough sub-groups for ~1.5 % of its source population firing in one step; when
    // the groups together want more than the budget, it is shared in proportion (work per step scales with
    // source size x row length, whatever the rates turn out to be).
    block = 0;
    const char *envBudget = getenv("GENNMI_PRESYN_BLOCKS_PER_CU");
    const uint32_t blocksPerCU = envBudget ? std::max(1, atoi(envBudget)) : 4u;
    // the launch has one grid row per batch, so the budget is per batch (at least one block per compute unit in all)
    const uint64_t budget = std::max<uint64_t>((numCU + r->batch - 1) / r->batch, (uint64_t)numCU * blocksPerCU / r->batch);
    std::vector<uint64_t> wantBlocks;
    for(auto &p : r->pre) {
        const uint32_t rowLen = (p.g.matrix == GENNMI_MATRIX_SPARSE) ? p.g.rowStride : (uint32_t)(p.g.conv[0] * p.g.conv[1] * p.g.conv[7]);
        uint32_t W;
        if(p.g.span == GENNMI_SPAN_PRE) { W = std::min(64u, pow2Ceil(std::max(1u, p.g.numThreadsPerSpike))); }
        else if(p.g.span == GENNMI_SPAN_POST) { W = WAVE; }
        else { W = std::min<uint32_t>(WAVE, std::max(4u, pow2Ceil((rowLen + 3) / 4))); }
        p.lanesPerSpike = W;
        p.vec4 = (p.g.matrix == GENNMI_MATRIX_SPARSE && p.g.wum != GENNMI_WUM_STDP_TRACE && (p.g.rowStride % 4) == 0
                  && (reinterpret_cast<uintptr_t>(p.g.ind) % 16) == 0 && (reinterpret_cast<uintptr_t>(p.g.g) % 16) == 0
                  && (p.g.wum != GENNMI_WUM_STATIC_PULSE_DENDRITIC_DELAY || (reinterpret_cast<uintptr_t>(p.g.d) % 4) == 0)
                  && W >= 16) ? 1u : 0u;
        const uint32_t span = W * (p.vec4 ? 4u : 1u);
        const uint64_t chunksPerRow = (rowLen + span - 1) / span;
        const uint64_t wantSubGroups = std::max<uint64_t>(8, ((uint64_t)p.g.numSrcNeurons * chunksPerRow) / 64);
        wantBlocks.push_back(std::min<uint64_t>((wantSubGroups * W + BLOCK - 1) / BLOCK, budget));
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
        const uint32_t cap = std::max(1u, (numCU * 16u) / (uint32_t)r->post.size());
        p.startBlock = block;
        p.numBlocks = std::max(1u, (uint32_t)std::min<uint64_t>((wantSubGroups * p.lanesPerSpike + BLOCK - 1) / BLOCK, cap));
        block += p.numBlocks;
    }
    r->postBlocks = block;

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
        const uint32_t tileFloats = envTile ? (uint32_t)std::max(0, atoi(envTile)) : 16384u;
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
               || (p.g.wum != GENNMI_WUM_STATIC_PULSE && p.g.wum != GENNMI_WUM_STDP_TRACE)) { continue; }
            const uint32_t tileSize = std::min(tileFloats, p.g.numTrgNeurons);
            const uint32_t numTiles = (p.g.numTrgNeurons + tileSize - 1) / tileSize;
            uint16_t *dOff = nullptr; uint32_t *dFlag = nullptr;
            HIP_TRY(hipMalloc(&dOff, (size_t)p.g.numSrcNeurons * (numTiles + 1) * sizeof(uint16_t)));
            r->owned.push_back(dOff);
            HIP_TRY(hipMalloc(&dFlag, sizeof(uint32_t)));
            HIP_TRY(hipMemset(dFlag, 0, sizeof(uint32_t)));
            tileOffsetKernel<<<dim3((p.g.numSrcNeurons + BLOCK - 1) / BLOCK), dim3(BLOCK), 0, 0>>>(
                p.g.numSrcNeurons, p.g.rowStride, p.g.rowLength, p.g.ind, tileSize, numTiles, dOff, dFlag);
            HIP_TRY(hipGetLastError());
            uint32_t unsorted = 0;
            HIP_TRY(hipMemcpy(&unsorted, dFlag, sizeof(uint32_t), hipMemcpyDeviceToHost));
            HIP_TRY(hipFree(dFlag));
            if(unsorted) { continue; }          // rows not sorted by target: the scatter kernel handles every step
            p.tileThreshold = std::max(1u, p.g.numTrgNeurons);
            const uint32_t avgSeg = std::max(1u, p.g.rowStride / numTiles);
            TileGroupDev t{};
            t.g = p.g; t.tileOff = dOff; t.numTiles = numTiles; t.tileSize = tileSize;
            const char *envLanes = getenv("GENNMI_TILE_LANES");
            t.lanes = envLanes ? std::min<uint32_t>(WAVE, pow2Ceil((uint32_t)std::max(1, atoi(envLanes)))) : std::min<uint32_t>(WAVE, pow2Ceil((avgSeg + 7) / 8));
            t.threshold = p.tileThreshold;
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
            for(auto &t : tileGroups) {
                const uint32_t numSplits = std::max(1u, std::min(256u, budget / t.numTiles));
                t.numSplits = numSplits;
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

    // ---- single-launch step: possible when every projection is a SPARSE dendritic-delay one with ring depth >= 2
    // and nothing is plastic
    bool anyEvents = false;
    for(const auto &n : r->neuron) { anyEvents = anyEvents || n.g.numSpkEvent != 0; }
    const char *envFused = getenv("GENNMI_FUSED_STEP");
    bool eligible = !(envFused && atoi(envFused) == 0) && !r->pre.empty() && r->post.empty() && r->dense.empty() && r->proc.empty() && !anyEvents && r->neuronsPerLane == 1;
    for(const auto &p : r->pre) {
        eligible = eligible && p.g.matrix == GENNMI_MATRIX_SPARSE && p.g.wum == GENNMI_WUM_STATIC_PULSE_DENDRITIC_DELAY
                   && p.g.maxDenDelay >= 2 && p.g.numSrcDelaySlots <= 1;
        bool found = false;
        for(const auto &n : r->neuron) { found = found || (n.g.spk == p.g.srcSpk && n.g.numNeurons == p.g.numSrcNeurons); }
        eligible = eligible && found;
    }
    if(eligible) {
        auto devAlloc = [r](void **q, size_t bytes) -> hipError_t {
            hipError_t e = hipMalloc(q, bytes ? bytes : 4);
            if(e == hipSuccess) { r->owned.push_back(*q); e = hipMemset(*q, 0, bytes ? bytes : 4); }
            return e;
        };
        for(auto &n : r->neuron) {
            HIP_TRY(devAlloc((void**)&n.shadowSpk, 2 * (size_t)r->batch * n.g.numNeurons * sizeof(uint32_t)));
            HIP_TRY(devAlloc((void**)&n.shadowCnt, 2 * (size_t)r->batch * sizeof(uint32_t)));
            std::vector<PreGroupDev*> outs;
            for(auto &p : r->pre) { if(p.g.srcSpk == n.g.spk) { outs.push_back(&p); } }
            if(outs.empty()) { continue; }
            const uint32_t N = n.g.numNeurons;
            const dim3 grid((N + BLOCK - 1) / BLOCK);
            uint32_t *dLen = nullptr;
            HIP_TRY(devAlloc((void**)&dLen, (size_t)N * sizeof(uint32_t)));
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
            HIP_TRY(devAlloc((void**)&dStart, (size_t)(N + 1) * sizeof(uint32_t)));
            HIP_TRY(hipMemcpy(dStart, start.data(), (size_t)(N + 1) * sizeof(uint32_t), hipMemcpyHostToDevice));
            HIP_TRY(devAlloc((void**)&dOffset, (size_t)N * sizeof(uint32_t)));
            HIP_TRY(devAlloc((void**)&dEntries, (size_t)std::max(1u, start[N]) * sizeof(ZeroDelayEntry)));
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
                HIP_TRY(hipMalloc((void**)&n.spikeBitmap, words * sizeof(uint32_t)));
                HIP_TRY(hipMemset(n.spikeBitmap, 0, words * sizeof(uint32_t)));
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
    HIP_TRY(uploadPerBlock(r->neuron, r->neuronBlocks, &r->dNeuron));
    HIP_TRY(uploadPerBlock(r->pre, r->preBlocks, &r->dPre));
    HIP_TRY(uploadPerBlock(r->post, r->postBlocks, &r->dPost));
    HIP_TRY(uploadPerBlock(r->dense, r->denseBlocks, &r->dDense));
    HIP_TRY(uploadPerBlock(r->proc, r->procBlocks, &r->dProc));
    const size_t aggCount = 2 * (size_t)r->neuronBlocks * r->batch;       // per-block counts, then per-group totals
    HIP_TRY(hipMalloc(&r->dAgg, aggCount * sizeof(unsigned long long)));
    HIP_TRY(hipMemset(r->dAgg, 0, aggCount * sizeof(unsigned long long)));
    { const int rc = setupResident(r, numCU); if(rc) { return rc; } }
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
    bool stale;
    {
        std::lock_guard<std::mutex> lock(g_runnersMutex);
        stale = r->sourcesStale;
        r->sourcesStale = false;
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
    if(timed) {
        if(r->pending.size() >= 2048) { const int rc = drainTimers(r); if(rc) { return rc; } }
        const int rc = stamp(r, &e0); if(rc) { return rc; }
    }
    if(!r->pre.empty() || r->denseBlocks || r->procBlocks) {
        if(r->procBlocks) {
            presynapticProceduralKernel<<<dim3(r->procBlocks, r->batch), dim3(BLOCK), 0, r->stream>>>(r->dProc, r->dEvents);
        }
        if(r->preBlocks) {
            presynapticUpdateKernel<<<dim3(r->preBlocks, r->batch), dim3(BLOCK), 0, r->stream>>>(r->dPre, a, r->dt, r->dEvents);
        }
        if(r->denseBlocks) {
            presynapticDenseKernel<<<dim3(r->denseBlocks, r->batch), dim3(BLOCK), 0, r->stream>>>(r->dDense, r->dEvents);
        }
        if(r->tileBlocks) {
            presynapticTileKernel<<<dim3(r->tileBlocks, r->batch), dim3(r->tileThreads), r->tileFloats * sizeof(float), r->stream>>>(r->dTile, a, r->dt, r->dEvents);
        }
        if(r->convTileBlocks) {
            presynapticConvTileKernel<<<dim3(r->convTileBlocks, r->batch), dim3(CONV_TILE_THREADS), r->convTileBytes, r->stream>>>(r->dConvTile, r->dEvents);
        }
        if(timed) { const int rc = stamp(r, &e1); if(rc) { return rc; } r->pending.push_back({e0, e1, 0}); }
    }
    if(!r->post.empty()) {
        postsynapticUpdateKernel<<<dim3(r->postBlocks), dim3(BLOCK), r->postLdsBytes, r->stream>>>(r->dPost, a, r->dt);
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

// one whole timestep: a single launch where the runner allows it, else synapse kernels then the neuron kernel
static int launchStep(gennmi_runner *r, const StepArgs &a)
{
    if(r->fusedStep) { return launchFusedStep(r, a); }
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

int gennmi_step(gennmi_runner *r, float t, uint32_t recordingTimestep)
{
    if(!r || !r->finalised) { return fail(GENNMI_ESTATE, "step: runner not finalised"); }
    { const int rc = refreshSpikeSources(r); if(rc) { return rc; } }
    if(r->fusedStep) {
        StepArgs a{};
        a.base = nullptr; a.epoch = r->epoch; a.t = t; a.recordingTimestep = recordingTimestep;
        hipEvent_t e0 = nullptr, e1 = nullptr;
        if(r->timing) {
            if(r->pending.size() >= 2048) { const int rc = drainTimers(r); if(rc) { return rc; } }
            const int rc = stamp(r, &e0); if(rc) { return rc; }
        }
        const int rc = launchFusedStep(r, a);
        if(rc) { return rc; }
        if(r->timing) { const int rc2 = stamp(r, &e1); if(rc2) { return rc2; } r->pending.push_back({e0, e1, 3}); }
        r->epoch++;
        return GENNMI_OK;
    }
    const int rc = gennmi_update_synapses(r, t);
    if(rc) { return rc; }
    return gennmi_update_neurons(r, t, recordingTimestep);
}

int gennmi_run_steps(gennmi_runner *r, unsigned long long timestep, unsigned long long numSteps, unsigned long long numRecordingTimesteps)
{
    if(!r || !r->finalised) { return fail(GENNMI_ESTATE, "run_steps: runner not finalised"); }
    { const int rc = refreshSpikeSources(r); if(rc) { return rc; } }
    constexpr unsigned long long CHUNK = 100;
    const StepState hs{timestep, r->epoch, numRecordingTimesteps};
    HIP_TRY(hipMemcpyAsync(r->dState, &hs, sizeof(hs), hipMemcpyHostToDevice, r->stream));
    HIP_TRY(hipStreamSynchronize(r->stream));   // hs lives on this stack frame
    unsigned long long done = 0;
    if(r->resident && !r->timing && numSteps >= 4) { return launchResident(r, timestep, numSteps, numRecordingTimesteps); }
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
    HIP_TRY(hipStreamSynchronize(r->stream));
    uint32_t err = 0;
    HIP_TRY(hipMemcpy(&err, r->dError, sizeof(err), hipMemcpyDeviceToHost));
    if(err) { return fail(GENNMI_EDEVICE, "a kernel's bounded wait for other work-groups expired (spike offsets or spike exchange); state is undefined"); }
    return GENNMI_OK;
}

int gennmi_runner_set_timing(gennmi_runner *r, int enabled)
{
    if(!r) { return fail(GENNMI_EINVAL, "runner_set_timing: null runner"); }
    if(!enabled) { const int rc = drainTimers(r); if(rc) { return rc; } }
    r->timing = (enabled != 0);
    return GENNMI_OK;
}

int gennmi_runner_get_times(gennmi_runner *r, double *neuronUpdateTime, double *presynapticUpdateTime, double *postsynapticUpdateTime)
{
    if(!r) { return fail(GENNMI_EINVAL, "runner_get_times: null runner"); }
    { const int rc = drainTimers(r); if(rc) { return rc; } }
    if(neuronUpdateTime) { *neuronUpdateTime = r->neuronTime; }
    if(presynapticUpdateTime) { *presynapticUpdateTime = r->preTime; }
    if(postsynapticUpdateTime) { *postsynapticUpdateTime = r->postTime; }
    return GENNMI_OK;
}

int gennmi_runner_kernel_stats(gennmi_runner *r, double stats[8])
{
    if(!r || !stats) { return fail(GENNMI_EINVAL, "runner_kernel_stats: null argument"); }
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
    info[0] = (r->fusedStep ? 1u : 0u) | (r->resident ? 2u : 0u) | (r->neuronsPerLane > 1 ? 4u : 0u); info[1] = r->neuronBlocks; info[2] = r->preBlocks; info[3] = r->postBlocks;
    return GENNMI_OK;
}

int gennmi_runner_event_count(gennmi_runner *r, unsigned long long *events)
{
    if(!r || !events) { return fail(GENNMI_EINVAL, "runner_event_count: null argument"); }
    HIP_TRY(hipStreamSynchronize(r->stream));
    HIP_TRY(hipMemcpy(events, r->dEvents, sizeof(*events), hipMemcpyDeviceToHost));
    return GENNMI_OK;
}

int gennmi_max_col_length(uint32_t numSrc, uint32_t numTrg, uint32_t rowStride, const uint32_t *rowLength, const uint32_t *ind, uint32_t *maxColLength)
{
    if(!rowLength || !ind || !maxColLength || rowStride == 0) { return fail(GENNMI_EINVAL, "max_col_length: bad arguments"); }
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

int gennmi_build_remap(uint32_t numSrc, uint32_t numTrg, uint32_t rowStride, uint32_t colStride,
                       const uint32_t *rowLength, const uint32_t *ind, uint32_t *colLength, uint32_t *remap)
{
    if(!rowLength || !ind || !colLength || !remap || rowStride == 0 || colStride == 0) { return fail(GENNMI_EINVAL, "build_remap: bad arguments"); }
    if(colStride > REMAP_SORT_MAX) { return fail(GENNMI_EUNSUPPORTED, "build_remap: column stride above 16384 is not supported"); }
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
    const size_t lds = (size_t)pow2Ceil(colStride) * sizeof(uint32_t);
    if(lds > 48 * 1024) {
        HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void*>(remapSortKernel), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    }
    remapSortKernel<<<dim3(numTrg), dim3(BLOCK), lds, 0>>>(colStride, colLength, remap);
    HIP_TRY(hipGetLastError());
    HIP_TRY(hipDeviceSynchronize());
    return GENNMI_OK;
}

}   // extern "C"
