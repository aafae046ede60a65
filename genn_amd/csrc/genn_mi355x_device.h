// Part of libgenn_mi355x.so: included by genn_mi355x.hip only (one translation unit).
#ifndef GENN_MI355X_DEVICE_H
#define GENN_MI355X_DEVICE_H

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
    uint32_t *spikeBitmap;              // [batch][ceil(N/32)] engine-private bitmap of this step's spikes (populations at either end of a plastic projection), or NULL
    size_t bitmapStride;                // != 0: two bitmaps this many words apart; the update after k completed steps writes copy (k + 1) & 1, so that a
                                        //       kernel of the same launch can still read the spikes of the step before (copy k & 1)
    unsigned long long *aggEvent;       // look-back area of the spike-like event queues (groups with events), or NULL
    float *nextSpikeTime;               // spike sources: engine-private copy of spikeTimes[startSpike] per neuron (+inf: none left)
    size_t spikeTimesBytes;             // spike sources: bytes from spikeTimes to the end of its allocation (host bookkeeping)
};

// The learnPost half of a plastic projection, as its presynaptic half needs it.  The reference runs the presynaptic update of
// every projection, then the postsynaptic one (backendSIMT.cc genPresynapticUpdateKernel / genPostsynapticUpdateKernel,
// launched one after the other): a synapse whose two ends both fired in the last neuron update gets the presynaptic-spike
// rule first and the postsynaptic-spike rule second.  Here the thread that applies the first rule to such a synapse also
// applies the second, and the postsynaptic pass leaves every synapse of a row whose neuron fired to it — each synapse has
// one writer per step, the order on it is the reference's, and the two passes need not wait for each other.
struct LearnPostDev
{
    const float *srcST, *preTrace;      // [batch][numSrc] the postsynaptic-spike rule's view of the source neurons
    const uint32_t *trgBitmap;          // [batch][ceil(numTrg/32)] the target population's spikes of the last neuron update
    float aPlus, tauPlus;
    uint32_t enabled;                   // 0: the projection has no such partner, its presynaptic half is all there is
    uint32_t pad_;
};

struct PreGroupDev
{
    gennmi_presynaptic_update_group_t g;
    LearnPostDev learn;
    uint32_t startBlock, numBlocks;
    uint32_t lanesPerSpike;             // power of two, 1..64
    uint32_t vec4;                      // rows are 16-byte aligned and padded: dwordx4 loads
    int32_t convBH, convBW;
    uint32_t skipZeroDelay;             // synapses with d % D == 0 are delivered by the neuron update instead
    uint32_t tileThreshold;             // != 0: leave the step to the tile kernel when numSpikes*workPerSpike reaches it
    uint32_t workPerSpike;              // rowStride (SPARSE) or kh*kw*oc (Toeplitz)
    uint32_t ordered;                   // != 0: the projection is gathered by presynapticOrderedKernel, the scatter kernel leaves it alone
    const uint32_t *shadowSpk;          // the source population's shadow queue (read instead of srcSpk when set)
    const uint32_t *shadowCnt;
};

// Dense-activity path of a static SPARSE projection without delay: one block accumulates the events that
// fall into one tile of postsynaptic neurons in LDS and flushes the tile with lane-consecutive atomics.
struct TileGroupDev
{
    gennmi_presynaptic_update_group_t g;
    LearnPostDev learn;
    const uint16_t *tileOff;            // [numSrc*(numTiles+1)] first position of every row whose target is >= tile*tileSize
    uint32_t numTiles, tileSize;
    uint32_t tile, split, numSplits;    // this block: which tile, which share of the spikes
    uint32_t lanes;                     // lanes per (spike, tile) segment, power of two
    uint32_t threshold;
    uint32_t spikesPerSplit;            // a step's spikes are shared between max(2, numSpikes / spikesPerSplit) of a tile's blocks (record path)
    uint32_t recLanes;                  // != 0: the projection has segment records (below), read by this many lanes each (5 or 10)
    const uint8_t *records;             // [numTiles][numSrc] records of 24 * recLanes + 8 bytes (128 or 256), or NULL
    const uint8_t *overflow;            // [numTiles][numSrc] 64-byte records of the 8 synapses that follow a full record, or NULL
};
constexpr uint32_t REC_OVERFLOW = 8;    // synapses per overflow record: float weight[8], uint16_t target[8], 16 spare bytes

// Segment records: an engine-private copy of a static SPARSE projection in which the synapses of one (row, tile) segment
// form one record that starts on a cache-line boundary:
//     float    weight[4 * recLanes]        zero-filled beyond the segment
//     uint16_t target[4 * recLanes]        tile-local postsynaptic index
//     uint16_t count, first                synapses in the segment; position of the first one within its row
//     uint32_t spare
// A spike then costs each tile exactly one aligned line of 128 (256) bytes instead of two short reads at arbitrary offsets
// plus a look-up of the segment's boundaries.  The next 8 synapses of a segment longer than a record sit in a second,
// 64-byte record (read only by those segments: one more aligned read instead of two unaligned ones into the row); what
// exceeds both is read from the row itself.
__host__ __device__ constexpr uint32_t recordBytes(uint32_t recLanes) { return 24u * recLanes + 8u; }

// Dense-activity path of a Toeplitz Conv2D projection: a block owns rowsPerTile output rows (all columns and
// channels) in LDS next to a copy of the kernel weights.
struct ConvTileDev
{
    gennmi_presynaptic_update_group_t g;
    int32_t convBH, convBW;
    uint32_t rowsPerTile, tileRow0;
    uint32_t threshold, pad_;
};

// Dense path of a Toeplitz Conv2D projection on the matrix cores: at the activity that sends a step to a tile kernel, the
// layer is a small GEMM per batch — output pixels x (kh*kw*ic) x output channels — whose left operand is the source
// population's spike bitmap expanded to 0 / 1.
struct ConvMfmaDev
{
    gennmi_presynaptic_update_group_t g;
    const uint32_t *srcBitmap;          // [batch][ceil(numSrc/32)] the source population's spikes of the last neuron update
    int32_t convBH, convBW;
    uint32_t rowsPerBlock;              // output rows of a block
    uint32_t patchRows, patchPitch;     // the input patch of a block in LDS: [ic][patchRows][patchPitch] floats
    uint32_t planePitch;                // patchRows * patchPitch, padded
    uint32_t kernPitch;                 // the kernel in LDS: [kh*kw*ic, rounded up to whole chunks of steps][kernPitch] floats
    uint32_t threshold;
    uint32_t numBatches;                // the grid is one-dimensional: block = rowGroup * numBatches + batch
    uint32_t spikeWords;                // conv + neuron update in one kernel: words of a block's spike bitmap in LDS (behind patch and kernel)
    uint32_t restBlocks;                // ... and blocks of the other populations' updates, shared out between the layer's work-groups
    uint32_t restNeuronsPerLane, pad2_;
    size_t bitmapStride;                // see NeuronGroupDev::bitmapStride: after k completed steps the layer reads copy k & 1 of srcBitmap
};

struct PostGroupDev
{
    gennmi_postsynaptic_update_group_t g;
    uint32_t startBlock, numBlocks;
    uint32_t lanesPerSpike;
    uint32_t denseThreshold;            // != 0: steps with at least this many postsynaptic spikes walk the rows instead
    const uint32_t *spikeBitmap;        // [batch][ceil(numTrg/32)] this step's postsynaptic spikes, written by the neuron update
    const uint32_t *srcBitmap;          // [batch][ceil(numSrc/32)] != NULL: rows of neurons that fired are left to the presynaptic pass (LearnPostDev)
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
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4u __attribute__((ext_vector_type(4), aligned(4)));     // dword-aligned only: segments start anywhere in a row
typedef float f32x4u __attribute__((ext_vector_type(4), aligned(4)));

__device__ __forceinline__ void atomicAddF32(GLOBAL_AS float *addr, float v)
{
    // gfx950 has a native global_atomic_add_f32; the old value is not needed
    __builtin_amdgcn_global_atomic_fadd_f32(addr, v);
}

// fp32 add into LDS.  The native LDS float atomic of this part (ds_add_f32) retires one lane every three clocks per
// compute unit — 204 G adds/s for the whole chip, measured, whatever the addresses — while the integer path of the same
// banks sustains over 3,000 G/s; a compare-and-swap loop on that path adds floats at 1,450 to 1,600 G/s.  The sum is the
// same single fp32 addition either way.
__device__ __forceinline__ void ldsAddF32(float *addr, float v)
{
    uint32_t *p = reinterpret_cast<uint32_t*>(addr);
    uint32_t old = __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP), assumed;
    do {
        assumed = old;
        old = atomicCAS(p, assumed, __float_as_uint(__uint_as_float(assumed) + v));
    } while(old != assumed);
}

// The runner's error flag lives in pinned host memory that the device sees too: a bounded wait that expires stores 1 there
// (the flag only ever goes from 0 to 1, so a store does what an atomic OR would, on any kind of memory), and the host reads
// the word after waiting for the stream — no copy command behind every launch (3.5 us per launch and wait).
__device__ __forceinline__ void raiseErrorFlag(uint32_t *errorFlag)
{
    __hip_atomic_store(errorFlag, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
}

// The runner's count of synaptic events is kept as EVENT_SLOTS partial counts a cache line apart (the host adds them up):
// atomics on ONE address complete one after the other, about 8 ns each, so a launch whose thousand wavefronts each add
// their share to a single counter ends 8 us after its last useful instruction — and any barrier behind such an add waits
// that long.  A wavefront adds to the slot its work-group and wavefront numbers select.
constexpr uint32_t EVENT_SLOTS = 64, EVENT_SLOT_STRIDE = 16;        // (16 x 8 bytes = 128 bytes)
__device__ __forceinline__ void addEvents(unsigned long long *eventCounter, unsigned long long events)
{
    const uint32_t slot = (blockIdx.x * 5u + blockIdx.y * 3u + (threadIdx.x / WAVE)) & (EVENT_SLOTS - 1);
    atomicAdd(&eventCounter[(size_t)slot * EVENT_SLOT_STRIDE], events);
}

// four adds of one lane with their LDS round trips overlapped: all reads, then all swaps, then whatever lost a race
// (including two of the four that name the same element) one by one.  Straight-line code: an add that is switched off
// goes to a word of the lane's own instead of being branched around — with a branch per add the compiler waits for each
// swap before it issues the next, five dependent LDS round trips and a dozen changes of the execution mask per call, which
// is what bounded the tile kernels' main loops (a wavefront's pass, not memory, set their pace).
__device__ __forceinline__ float *ldsOwnWord()
{
    __shared__ float unused[1024];          // (one word per thread of the largest work-group)
    return &unused[threadIdx.x];
}

__device__ __forceinline__ void ldsAddF32x4(float *a0, float v0, bool p0, float *a1, float v1, bool p1, float *a2, float v2, bool p2, float *a3, float v3, bool p3)
{
    float *own = ldsOwnWord();
    uint32_t *q0 = reinterpret_cast<uint32_t*>(p0 ? a0 : own), *q1 = reinterpret_cast<uint32_t*>(p1 ? a1 : own);
    uint32_t *q2 = reinterpret_cast<uint32_t*>(p2 ? a2 : own), *q3 = reinterpret_cast<uint32_t*>(p3 ? a3 : own);
    const uint32_t o0 = __hip_atomic_load(q0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    const uint32_t o1 = __hip_atomic_load(q1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    const uint32_t o2 = __hip_atomic_load(q2, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    const uint32_t o3 = __hip_atomic_load(q3, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    __builtin_amdgcn_sched_barrier(0);      // (all four reads are issued before the first swap waits for its own)
    const uint32_t r0 = atomicCAS(q0, o0, __float_as_uint(__uint_as_float(o0) + v0));
    const uint32_t r1 = atomicCAS(q1, o1, __float_as_uint(__uint_as_float(o1) + v1));
    const uint32_t r2 = atomicCAS(q2, o2, __float_as_uint(__uint_as_float(o2) + v2));
    const uint32_t r3 = atomicCAS(q3, o3, __float_as_uint(__uint_as_float(o3) + v3));
    __builtin_amdgcn_sched_barrier(0);
    if(((r0 ^ o0) | (r1 ^ o1) | (r2 ^ o2) | (r3 ^ o3)) != 0u) {
        if(r0 != o0) { ldsAddF32(reinterpret_cast<float*>(q0), v0); }
        if(r1 != o1) { ldsAddF32(reinterpret_cast<float*>(q1), v1); }
        if(r2 != o2) { ldsAddF32(reinterpret_cast<float*>(q2), v2); }
        if(r3 != o3) { ldsAddF32(reinterpret_cast<float*>(q3), v3); }
    }
}

// the same for two adds
__device__ __forceinline__ void ldsAddF32x2(float *a0, float v0, bool p0, float *a1, float v1, bool p1)
{
    float *own = ldsOwnWord();
    uint32_t *q0 = reinterpret_cast<uint32_t*>(p0 ? a0 : own), *q1 = reinterpret_cast<uint32_t*>(p1 ? a1 : own);
    const uint32_t o0 = __hip_atomic_load(q0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    const uint32_t o1 = __hip_atomic_load(q1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    const uint32_t r0 = atomicCAS(q0, o0, __float_as_uint(__uint_as_float(o0) + v0));
    const uint32_t r1 = atomicCAS(q1, o1, __float_as_uint(__uint_as_float(o1) + v1));
    if(((r0 ^ o0) | (r1 ^ o1)) != 0u) {
        if(r0 != o0) { ldsAddF32(reinterpret_cast<float*>(q0), v0); }
        if(r1 != o1) { ldsAddF32(reinterpret_cast<float*>(q1), v1); }
    }
}

}   // namespace

#endif
