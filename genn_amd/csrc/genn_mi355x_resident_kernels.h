// Part of libgenn_mi355x.so: included by genn_mi355x.hip only (one translation unit).
#ifndef GENN_MI355X_RESIDENT_KERNELS_H
#define GENN_MI355X_RESIDENT_KERNELS_H


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
constexpr uint32_t RES_SEQ_MASK = (1u << (64 - RES_SEQ_SHIFT)) - 1u;    // sequence numbers run on from launch to launch, modulo 2^23
constexpr uint32_t RES_WORD_IDS = 4;         // spikes of a tile and step that travel inside its word (more: side buffer)
constexpr uint32_t RES_REPLICAS = 8;         // copies of the word array, one per XCD, so that polling spreads over memory channels

struct ResProj
{
    const u32x2 *packed;                // one record per (padded) synapse, see residentPackKernel
    const u32x4 *seg;                   // [numSrc * tilesInGroup][2]: the row's part inside a tile, see residentSegKernel
    uint32_t D;                         // ring depth; 0 = no dendritic delay, events add to inSyn
    uint32_t lds;                       // float offset of the ring (D x RES_T, slot-major) or inSyn row in the tile's LDS
    uint32_t srcGroup;
    uint32_t magic;                     // floor(2^32 / D) + 1: x % D for x < 2^16 is x - mulhi(x, magic) * D
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

// The synapses as the row walk reads them: target inside its tile | dendritic delay << 8, and the weight's bits — one
// 8-byte load per synapse instead of three loads from three arrays (three pages, three cache lines per row part).
// Same index as the arrays it is made from; padding beyond a row's length is copied as it is and never read.
__global__ void residentPackKernel(size_t numSynapses, const uint32_t *ind, const float *weight, const uint8_t *delay, u32x2 *packed)
{
    const size_t id = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if(id >= numSynapses) { return; }
    u32x2 rec;
    rec.x = (ind[id] & (RES_T - 1)) | (delay ? (uint32_t)delay[id] << 8 : 0u); rec.y = __float_as_uint(weight[id]);
    packed[id] = rec;
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

// POISSON: some population has a PoissonExp current source (its state then lives in a register per source and neuron);
// the instantiation without it carries neither the registers nor the generator
template<bool POISSON>
__global__ __launch_bounds__(BLOCK)
void residentKernel(const ResTile * __restrict__ tiles, uint32_t numTiles, const NeuronGroupDev * __restrict__ groups,
                    const uint8_t * __restrict__ tileGroup, unsigned long long *tags, unsigned long long *side,
                    unsigned long long timestep0, unsigned long long epoch0, unsigned long long numRecordingTimesteps, uint32_t numSteps,
                    float dt, uint32_t zeroDelaySplit, uint32_t *errorFlag, unsigned long long *eventCounter, uint32_t replicaStride,
                    unsigned long long seqBase)
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

    // (a runner whose error flag is raised launches nothing more: the host looks at the flag before every launch; the flag
    // is host memory, and reading it here would put a trip over the bus in front of every launch)
    if(tid == 0) { shScalar[3] = 0u; }
    __syncthreads();

    // ---- tables into LDS
    for(uint32_t k = tid; k < numTiles; k += BLOCK) { shTileGroup[k] = tileGroup[k]; }
    const uint32_t numProj = T.numProj;
    if(tid < numProj) { shProj[tid] = T.proj[tid]; }
    __syncthreads();
    // projections grouped by source group (a counting sort of a handful of entries, read from the LDS copy; every thread
    // finds one entry's place by itself — one thread doing all of it is a chain of a hundred dependent LDS reads, 3 us
    // of every launch)
    if(tid <= RES_MAX_GROUPS) {
        uint32_t below = 0;
        for(uint32_t q = 0; q < numProj; q++) { below += (shProj[q].srcGroup < tid) ? 1u : 0u; }
        shProjStart[tid] = below;
    }
    if(tid < numProj) {
        const uint32_t s = shProj[tid].srcGroup;
        uint32_t below = 0, before = 0;
        for(uint32_t q = 0; q < numProj; q++) {
            const uint32_t sq = shProj[q].srcGroup;
            below += (sq < s) ? 1u : 0u;
            before += (q < tid && sq == s) ? 1u : 0u;
        }
        shProjIdx[below + before] = (uint8_t)tid;
    }

    // ---- state: neuron variables in registers, inSyn and ring slices in LDS
    float l0 = 0, l1 = 0;
    if(mine) { l0 = asGlobal(g.var0)[i]; l1 = asGlobal(g.var1)[i]; }
    // state of the PoissonExp sources, in registers like the neuron's own
    float csState[GENNMI_MAX_CS];
    #pragma unroll
    for(uint32_t c = 0; c < GENNMI_MAX_CS; c++) {
        csState[c] = (POISSON && mine && c < numCS && g.cs[c].kind == GENNMI_CS_POISSON_EXP) ? asGlobal(g.cs[c].current)[i] : 0.0f;
    }
    for(uint32_t m = 0; m < numPSM; m++) {
        lds[T.ldsIn[m] + tid] = mine ? asGlobal(g.psm[m].outPost)[i] : 0.0f;
        const uint32_t D = g.psm[m].maxDenDelay;
        // (sixteen slots' loads in flight at a time: one at a time, a ring of 43 slots is 43 memory round trips per launch)
        GLOBAL_AS const float *ring = asGlobal(g.psm[m].denDelay) + (mine ? i : 0u);
        for(uint32_t slot0 = 0; slot0 < D; slot0 += 16) {
            float v[16];
            #pragma unroll
            for(uint32_t u = 0; u < 16; u++) { v[u] = (mine && slot0 + u < D) ? ring[(size_t)min(slot0 + u, D - 1) * n] : 0.0f; }
            #pragma unroll
            for(uint32_t u = 0; u < 16; u++) { if(slot0 + u < D) { lds[T.ldsRing[m] + (slot0 + u) * RES_T + tid] = v[u]; } }
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
    // A word slot is rewritten every second sequence number, and a launch continues the numbering of the one before
    // (seqBase), so a slot never holds the number a reader waits for before its writer has stored it: nothing is cleared
    // between launches.  A tile's spikes beyond those its word holds go through the side buffer, one 64-bit entry each that
    // says which exchange it belongs to (the unwrapped sequence number, 56 bits, above the tile-local index): entries and
    // word are stored in any order without a fence, and a reader that finds the word first waits for the entries.
    auto publish = [&](uint32_t step, uint32_t count) {
        const uint32_t seq = (uint32_t)((seqBase + step) & RES_SEQ_MASK);
        const uint32_t parity = seq & 1u;
        if(count > RES_WORD_IDS) {
            for(uint32_t r = tid; r < count; r += BLOCK) {
                __hip_atomic_store(&side[((size_t)parity * numTiles + blockIdx.x) * RES_T + r], ((seqBase + step) << 8) | (shOwn[r] - T.first),
                                   __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
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
    // Entries e0 .. e0 + 7 (below c) of a tile's side list of the exchange `full`: waits, bounded, until each says so
    auto sideIds = [&](uint32_t tile, uint32_t e0, uint32_t c, unsigned long long full, uint32_t parity, uint32_t (&local)[8]) -> bool {
        const unsigned long long *base = side + ((size_t)parity * numTiles + tile) * RES_T + e0;
        const unsigned long long want = full & 0x00FFFFFFFFFFFFFFull;
        uint32_t need = (c - e0 >= 8) ? 0xFFu : (1u << (c - e0)) - 1u, spins = 0;
        unsigned long long v[8];
        while(true) {
            #pragma unroll
            for(uint32_t u = 0; u < 8; u++) { v[u] = 0; if(need & (1u << u)) { v[u] = __hip_atomic_load(base + u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); } }
            #pragma unroll
            for(uint32_t u = 0; u < 8; u++) {
                if((need & (1u << u)) && (v[u] >> 8) == want) { local[u] = (uint32_t)v[u] & 0xFFu; need &= ~(1u << u); }
            }
            if(!need) { return true; }
            if(++spins > c_spinLimit) { return false; }
            __builtin_amdgcn_s_sleep(1);
        }
    };
    auto poll = [&](uint32_t step, unsigned long long epoch) -> bool {
        const uint32_t seq = (uint32_t)((seqBase + step) & RES_SEQ_MASK);
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
        if(!ok) { shScalar[3] = 1u; }                  // (zero since the launch began: a launch that finds the error flag raised has left)
        __syncthreads();
        if(shScalar[3]) {
            if(tid == 0) { raiseErrorFlag(errorFlag); }
            return false;
        }
        // front slot of every projection's ring in the step this exchange feeds
        if(tid < numProj) { shProjPtr[tid] = shProj[tid].D ? modStep(epoch + 1, shProj[tid].D) : 0u; }
        #pragma unroll
        for(uint32_t q = 0; q < WATCH; q++) {
            const uint32_t c = (uint32_t)(word[q] >> 32) & 0x1FFu, np = watchNumProj[q];
            if(c == 0 || np == 0) { continue; }
            uint32_t pos = atomicAdd(&shScalar[0], c * np);
            const bool fits = pos + c * np <= RES_PAIR_CAP;
            if(c <= RES_WORD_IDS) {
                for(uint32_t e = 0; fits && e < c; e++) {
                    const uint32_t id = watchFirst[q] + (((uint32_t)word[q] >> (8 * e)) & 0xFFu);
                    for(uint32_t j = 0; j < np; j++) { shPair[pos++] = make_uint2(id, shProjIdx[watchProj0[q] + j]); }
                }
                continue;
            }
            // a longer list: its entries, eight loads at a time (also when the pairs do not fit and the chunked walk will
            // read the list again: once seen here, an entry is there for every later read of this work-group)
            for(uint32_t e0 = 0; e0 < c && ok; e0 += 8) {
                uint32_t local[8];
                if(!sideIds(tid + q * BLOCK, e0, c, seqBase + step, parity, local)) { ok = false; break; }
                #pragma unroll
                for(uint32_t u = 0; u < 8; u++) {
                    if(!fits || e0 + u >= c) { continue; }
                    for(uint32_t j = 0; j < np; j++) { shPair[pos++] = make_uint2(watchFirst[q] + local[u], shProjIdx[watchProj0[q] + j]); }
                }
            }
        }
        if(!ok) { shScalar[3] = 1u; }
        __syncthreads();
        if(shScalar[3]) {
            if(tid == 0) { raiseErrorFlag(errorFlag); }
            return false;
        }
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

    // Walks the row segments of the staged pairs: a group of lanes per pair, a lane taking every n-th synapse of its
    // pair's segment, eight of them per trip to memory.  Sixteen lanes per pair when the pairs are few (a quiet step: one
    // trip covers 128 synapses of each of a wavefront's four pairs), four when they are many (a synchronous burst).
    // (Segments of a tile are short — a row's share of 256 targets — so lanes idle in the longest segment's last trip
    // cost less than finding, for every lane, its place in a list of all the segments' synapses would.)
    // A synapse is "due" when it lands in the slot read this step (delay a multiple of the ring depth, or no ring).
    // PASS_ALL adds every synapse, PASS_LATER those not due, PASS_DUE the due ones; `flaggedOnly` restricts the walk to
    // segments whose due synapses are not all inline in their entry.
    auto process = [&](uint32_t numPairs, uint32_t pass, bool flaggedOnly) {
        constexpr uint32_t TRIP = 8;
        const uint32_t shift = (numPairs <= 4 * (BLOCK / WAVE)) ? 4u : (numPairs <= 8 * (BLOCK / WAVE)) ? 3u : 2u;
        const uint32_t lanesPerPair = 1u << shift, pairsPerGroup = WAVE >> shift;
        for(uint32_t q0 = wave * pairsPerGroup; q0 < numPairs; q0 += (BLOCK / WAVE) * pairsPerGroup) {
            const uint32_t q = q0 + (lane >> shift);
            uint32_t len = 0, start = 0, proj = 0;
            if(q < numPairs) {
                const uint2 sg = shSeg[q];
                proj = shPair[q].y;
                const bool flagged = (sg.y & (RES_SEG_OVERFLOW | RES_SEG_NO_DELAY)) != 0;
                const bool skip = (flaggedOnly && !flagged) || (pass == PASS_LATER && (sg.y & RES_SEG_NO_DELAY));
                start = sg.x; len = skip ? 0u : (sg.y & 0xFFFFu);
            }
            const ResProj &P = shProj[proj];
            const uint32_t depth = P.D, front = shProjPtr[proj], ldsBase = P.lds, magic = P.magic;
            GLOBAL_AS const u32x2 *packed = asGlobal(P.packed) + start;
            for(uint32_t i0 = lane & (lanesPerPair - 1); __any(i0 < len); i0 += TRIP * lanesPerPair) {
                u32x2 rec[TRIP];
                #pragma unroll
                for(uint32_t u = 0; u < TRIP; u++) {
                    const uint32_t i = i0 + u * lanesPerPair;
                    rec[u].x = 0x80000000u; rec[u].y = 0u;               // (no synapse)
                    if(i < len) { rec[u] = packed[i]; }
                }
                #pragma unroll
                for(uint32_t u = 0; u < TRIP; u++) {
                    if(rec[u].x >> 31) { continue; }
                    const uint32_t x = front + (rec[u].x >> 8);              // far below 2^16: the ring fits the LDS, a delay is a byte
                    const uint32_t slot = depth ? x - __umulhi(x, magic) * depth : 0u;
                    const bool due = !depth || (slot == front);
                    if((pass == PASS_LATER && due) || (pass == PASS_DUE && !due)) { continue; }
                    unsafeAtomicAdd(&lds[ldsBase + slot * RES_T + (rec[u].x & 0xFFu)], __uint_as_float(rec[u].y));
                }
            }
        }
    };

    // the pairs of a step that holds more of them than shPair does: staged and walked RES_PAIR_CAP at a time, in full
    auto processChunked = [&](uint32_t step, uint32_t total, uint32_t pass, bool count) {
        const uint32_t parity = (seqBase + step) & 1u;
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
                                                            : tiles[k].first + ((uint32_t)__hip_atomic_load(&side[((size_t)parity * numTiles + k) * RES_T + q], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) & 0xFFu);
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
        if(convention != PASS_LATER && shFlagged) { process(total, PASS_DUE, true); __syncthreads(); }
        return (convention == PASS_DUE) ? 0u : total;
    };
    // the rest of those pairs' synapses: none of them is read before the next step
    auto deliverLater = [&](uint32_t numPairs) {
        if(numPairs) { process(numPairs, PASS_LATER, false); }
    };

    // What the update reads of its group and tile, once: through the references every step would load it again (the
    // compiler cannot tell that nobody writes those structures while the kernel runs).
    float psmInit[GENNMI_MAX_PSM], psmDecay[GENNMI_MAX_PSM], csAmp[GENNMI_MAX_CS], par[8];
    uint32_t psmKind[GENNMI_MAX_PSM], psmDepth[GENNMI_MAX_PSM], psmIn[GENNMI_MAX_PSM], psmRing[GENNMI_MAX_PSM], csKind[GENNMI_MAX_CS];
    #pragma unroll
    for(uint32_t m = 0; m < GENNMI_MAX_PSM; m++) {
        const bool on = m < numPSM;
        psmInit[m] = on ? g.psm[m].init : 0.0f; psmDecay[m] = on ? g.psm[m].expDecay : 0.0f;
        psmKind[m] = on ? g.psm[m].kind : 0u; psmDepth[m] = on ? g.psm[m].maxDenDelay : 0u;
        psmIn[m] = on ? T.ldsIn[m] : 0u; psmRing[m] = on ? T.ldsRing[m] : 0u;
    }
    #pragma unroll
    for(uint32_t c = 0; c < GENNMI_MAX_CS; c++) { csAmp[c] = (c < numCS) ? g.cs[c].amp : 0.0f; csKind[c] = (c < numCS) ? g.cs[c].kind : 0u; }
    #pragma unroll
    for(uint32_t q = 0; q < 8; q++) { par[q] = g.params[q]; }
    const uint32_t neuronModel = g.model;
    uint32_t * const recordSpk = g.recordSpk;

    // ---- exchange the spikes that precede the first step, then step
    publish(1u, ownCount);
    bool ok = true;
    uint32_t k = 0;
    for(; k < numSteps; k++) {
        const unsigned long long epoch = epoch0 + k;
        if(!poll(k + 1, epoch)) { ok = false; break; }
        const uint32_t later = deliverDue(k + 1, (zeroDelaySplit && k == 0) ? PASS_LATER : PASS_ALL);     // (ends with a barrier)

        // neuron update: same operations in the same order as neuronBody
        bool spiked = false;
        if(mine) {
            float Isyn = 0;
            #pragma unroll
            for(uint32_t m = 0; m < GENNMI_MAX_PSM; m++) {
                if(m < numPSM) {
                    float linSyn = lds[psmIn[m] + tid];
                    const uint32_t D = psmDepth[m];
                    if(D) {
                        const uint32_t front = psmRing[m] + modStep(epoch + 1, D) * RES_T + tid;
                        linSyn += lds[front];
                        lds[front] = 0.0f;
                    }
                    if(psmKind[m] == GENNMI_PSM_EXPCURR) {
                        Isyn += psmInit[m] * linSyn;
                        linSyn *= psmDecay[m];
                    }
                    else {
                        Isyn += linSyn;
                        linSyn = 0.0f;
                    }
                    lds[psmIn[m] + tid] = linSyn;
                }
            }
            #pragma unroll
            for(uint32_t c = 0; c < GENNMI_MAX_CS; c++) {
                if(c < numCS) { Isyn += (!POISSON || csKind[c] == GENNMI_CS_DC) ? csAmp[c] : poissonExpStep(g.cs[c], csState[c], i, epoch); }
            }
            if(neuronModel == GENNMI_NEURON_LIF) {
                if(l1 <= 0.0f) {
                    const float alpha = ((Isyn + par[0]) * par[1]) + par[2];
                    l0 = alpha - (par[3] * (alpha - l0));
                }
                else {
                    l1 -= dt;
                }
                spiked = (l1 <= 0.0f && l0 >= par[4]);
                if(spiked) { l0 = par[5]; l1 = par[6]; }
            }
            else {
                if(l0 >= 30.0f) {
                    l0 = par[2];
                    l1 += par[3];
                }
                l0 += 0.5f * (0.04f * l0 * l0 + 5.0f * l0 + 140.0f - l1 + Isyn) * dt;
                l0 += 0.5f * (0.04f * l0 * l0 + 5.0f * l0 + 140.0f - l1 + Isyn) * dt;
                l1 += par[0] * (par[1] * l0 - l1) * dt;
                if(l0 > 30.0f) { l0 = 30.0f; }
                spiked = (l0 >= 29.99f);
            }
        }
        const unsigned long long ballot = __ballot(spiked);
        const uint32_t laneRank = __popcll(ballot & ((1ull << lane) - 1ull));
        if(lane == 0) { shWave[wave] = __popcll(ballot); }
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
        // while the words of this step travel: the step's recording words, and the synapses of the previous step's spikes
        // that are not due yet
        if(recordSpk && (lane & 31) == 0 && mine) {
            const unsigned long long ts = timestep0 + k;
            const uint32_t recT = numRecordingTimesteps ? (((ts | numRecordingTimesteps) >> 32) ? (uint32_t)(ts % numRecordingTimesteps)
                                                                                                : ((uint32_t)ts % (uint32_t)numRecordingTimesteps)) : 0u;
            recordSpk[(size_t)recT * ((n + 31) / 32) + (i >> 5)] = (uint32_t)(ballot >> (lane & 32));
        }
        deliverLater(later);
    }

    // ---- after the last step: everybody's last spikes give the position of this tile's spikes in the population's
    // queue; a runner that delivers front-slot synapses one step early (single-launch plan) wants them in the ring now
    const unsigned long long epochEnd = epoch0 + numSteps;       // completed steps
    if(ok && !poll(numSteps + 1, epochEnd)) { ok = false; }
    if(!ok) { return; }
    if(zeroDelaySplit) { deliverDue(numSteps + 1, PASS_DUE); }
    __syncthreads();

    if(mine) {
        asGlobal(g.var0)[i] = l0; asGlobal(g.var1)[i] = l1;
        #pragma unroll
        for(uint32_t c = 0; c < GENNMI_MAX_CS; c++) {
            if(POISSON && c < numCS && g.cs[c].kind == GENNMI_CS_POISSON_EXP) { asGlobal(g.cs[c].current)[i] = csState[c]; }
        }
    }
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
    if(lane == 0 && events) { addEvents(eventCounter, events); }
}


#endif
