// Part of libgenn_mi355x.so: included by genn_mi355x.hip only (one translation unit).
#ifndef GENN_MI355X_SYNAPSE_KERNELS_H
#define GENN_MI355X_SYNAPSE_KERNELS_H

namespace
{
// The postsynaptic-spike rule on one synapse (pygenn/genn_model.py:1464-1471 for the trace rule, weightUpdateModels.h:360-366
// for the built-in additive one), with the arithmetic of postsynapticUpdateKernel: used by the presynaptic passes for synapses
// whose target fired in the last neuron update as well (see LearnPostDev).
__device__ __forceinline__ float learnPostOnSynapse(const LearnPostDev &L, const gennmi_presynaptic_update_group_t &g, uint32_t batch,
                                                    uint32_t idPre, float w, float t, float dt, bool &changed)
{
    const size_t pre = (size_t)batch * g.numSrcNeurons + idPre;
    const float stPre = dt + asGlobal(L.srcST)[pre];
    const float dtSpike = t - stPre;
    if(dtSpike > 0) {
        const float factor = (L.tauPlus > 0.0f) ? (float)exp((double)(-dtSpike / L.tauPlus)) : asGlobal(L.preTrace)[pre];
        changed = true;
        return fminf(g.wMax, fmaxf(g.wMin, w + (L.aPlus * factor)));
    }
    return w;
}
// the same rule with what it reads of the presynaptic neuron (last spike time, trace) already in registers: the same for every
// synapse of a row
__device__ __forceinline__ float learnPostOnSynapseWith(const LearnPostDev &L, const gennmi_presynaptic_update_group_t &g, float stRaw, float trace,
                                                        float w, float t, float dt)
{
    const float stPre = dt + stRaw;
    const float dtSpike = t - stPre;
    if(dtSpike > 0) {
        const float factor = (L.tauPlus > 0.0f) ? (float)exp((double)(-dtSpike / L.tauPlus)) : trace;
        return fminf(g.wMax, fmaxf(g.wMin, w + (L.aPlus * factor)));
    }
    return w;
}
__device__ __forceinline__ bool bitmapTest(GLOBAL_AS const uint32_t *bitmap, uint32_t i) { return (bitmap[i >> 5] >> (i & 31)) & 1u; }

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
__device__ __forceinline__ void presynapticBody(const PreGroupDev &G, uint32_t blockInKernel, uint32_t batch, uint32_t numBatches,
                                                const Resolved &st, float dt, unsigned long long *eventCounter)
{
    const gennmi_presynaptic_update_group_t &g = G.g;
    if(G.ordered) { return; }
    const uint32_t W = G.lanesPerSpike;
    const uint32_t localBlock = blockInKernel - G.startBlock;
    const uint32_t lis = threadIdx.x & (W - 1);
    const uint32_t subGroup = (localBlock * blockDim.x + threadIdx.x) / W;      // (any multiple of the wavefront size will do as block size)
    const uint32_t numSubGroups = (G.numBlocks * blockDim.x) / W;
    // spikes of the previous step: the population's own queue, or (when this launch may run next to the
    // neuron update that refills that queue) the shadow copy written one step ago
    const uint32_t parity = (uint32_t)((st.epoch + 1) & 1);
    // axonal delay: the source's queue is a ring of slots; this projection reads the slot written axonalDelaySteps + 1
    // updates ago, (spkQuePtr + slots - delay) % slots with spkQuePtr = epoch % slots (backendBase.cc:207-216)
    const uint32_t slots = max(1u, g.numSrcDelaySlots);
    const uint32_t readSlot = (slots > 1) ? modStep(st.epoch + slots - g.axonalDelaySteps, slots) : 0u;
    GLOBAL_AS const uint32_t *cntPtr = G.shadowSpk ? asGlobal(G.shadowCnt) + (size_t)parity * numBatches + batch
                                                   : asGlobal(g.srcSpkCnt) + ((size_t)batch * slots + readSlot);
    GLOBAL_AS const uint32_t *spk = G.shadowSpk ? asGlobal(G.shadowSpk) + ((size_t)parity * numBatches + batch) * g.numSrcNeurons
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
            else {
                // trace STDP presynaptic-spike code (pygenn/genn_model.py:1456-1463); every synapse of
                // the row is owned by exactly one lane, so the read-modify-write of g needs no atomic
                // (plastic weights, spike times and traces are per batch: VarAccess::READ_WRITE variables are duplicated).
                // Index and weight are read with the row's length, not after it (rows are padded: any j < rowStride is readable).
                GLOBAL_AS float *wPtr = weight + (size_t)batch * g.numSrcNeurons * g.rowStride + rowBase + j;
                uint32_t idPost = 0; float w = 0.0f;
                if(inRow) { idPost = ind[rowBase + j]; w = *wPtr; }
                if(j >= npost) { if(lis == 0 && chunk == 0) { events += npost; } continue; }
                const size_t post = (size_t)batch * numTrg + idPost;
                // (everything the rule reads of the target is asked for at once: one trip to memory after the index, not three)
                const float stRaw = asGlobal(g.trgST)[post];
                const float trace = (g.wum == GENNMI_WUM_STDP) ? 0.0f : asGlobal(g.postTrace)[post];
                const uint32_t firedBits = G.learn.enabled ? asGlobal(G.learn.trgBitmap)[(size_t)batch * ((numTrg + 31) / 32) + (idPost >> 5)] : 0u;
                const float stPost = dt + stRaw;   // st_post = DT*(backPropSteps+1) + trgST (synapseUpdateGroupMerged.cc:134-142)
                atomicAddF32(&outPost[idPost], w);
                const float dtSpike = st.t - stPost;
                float newWeight = w;
                bool changed = false;
                if(dtSpike > 0) {
                    // trace rule: the target's trace; built-in additive rule (weightUpdateModels.h:352-359): the exponential
                    // of the time since the target's last spike, evaluated in double and rounded once as the reference does
                    const float factor = (g.wum == GENNMI_WUM_STDP) ? (float)exp((double)(-dtSpike / g.tauMinus)) : trace;
                    newWeight = fminf(g.wMax, fmaxf(g.wMin, w - (g.aMinus * factor)));
                    changed = true;
                }
                if((firedBits >> (idPost & 31u)) & 1u) {
                    newWeight = learnPostOnSynapse(G.learn, g, batch, idPre, newWeight, st.t, dt, changed);
                }
                if(changed) { *wPtr = newWeight; }
            }
            if(lis == 0 && chunk == 0) { events += npost; }
        }
    }

    // one counter update per wave
    for(int off = WAVE / 2; off > 0; off >>= 1) { events += __shfl_down(events, off, WAVE); }
    if((threadIdx.x & (WAVE - 1)) == 0 && events) { addEvents(eventCounter, events); }
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
    if((threadIdx.x & (WAVE - 1)) == 0 && events) { addEvents(eventCounter, events); }
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
    if(lane == 0 && events) { addEvents(eventCounter, events); }
}

// ------------------------------------------------------------------------------------------------
// Tile kernel.  Scattered fp32 atomics cost one memory transaction each (≈20 G/s measured on this part,
// whatever the array size), lane-consecutive ones ≈280 G/s.  When a step carries enough events
// (numSpikes*rowStride >= numTrg), a block therefore owns a tile of postsynaptic neurons in LDS: it walks
// its share of the spike list, reads only the segment of each row that falls into its tile (rows are
// sorted by target; tileOff holds the segment boundaries), adds into LDS, and finally flushes the tile
// with consecutive lanes on consecutive addresses.
// ------------------------------------------------------------------------------------------------
// Record variant of the tile kernel's main loop (static weights): L lanes read one (spike, tile) record — four weights
// (16 bytes) and four tile-local targets (8 bytes) each, plus the record's count word — so a wavefront takes 64 / L records
// per pass, every one a single aligned line.  The block's share of the spike queue is dealt so that one pass of the block
// covers consecutive queue entries: the queue ascends, so the block walks its tile's record array front to back.
template<uint32_t L>
__device__ __forceinline__ unsigned long long tileRecordLoop(const TileGroupDev &G, GLOBAL_AS const uint32_t *spk, uint32_t numSpikes, uint32_t activeSplits,
                                                             float *shTile, uint32_t tileStart)
{
    constexpr uint32_t C = 4 * L, REC = recordBytes(L), GROUPS = WAVE / L;
    const gennmi_presynaptic_update_group_t &g = G.g;
    const uint32_t lane = threadIdx.x & (WAVE - 1);
    const uint32_t group = lane / L, k = lane % L;
    const bool live = group < GROUPS;
    const uint32_t perBlock = (blockDim.x / WAVE) * GROUPS;
    const uint32_t stride = perBlock * activeSplits;
    const uint32_t lastSrc = g.numSrcNeurons - 1;
    GLOBAL_AS const uint8_t *records = asGlobal(G.records) + (size_t)G.tile * g.numSrcNeurons * REC;
    GLOBAL_AS const uint8_t *overflow = G.overflow ? asGlobal(G.overflow) + (size_t)G.tile * g.numSrcNeurons * 64 : nullptr;
    unsigned long long events = 0;
    struct Rec { f32x4 w; uint32_t t01, t23, meta; };
    auto fetch = [&](uint32_t id) -> Rec {
        GLOBAL_AS const uint8_t *rec = records + (size_t)id * REC;
        Rec r;
        r.w = *reinterpret_cast<GLOBAL_AS const f32x4*>(rec + 16 * k);
        const u32x2 t = *reinterpret_cast<GLOBAL_AS const u32x2*>(rec + 16 * L + 8 * k);
        r.t01 = t.x; r.t23 = t.y;
        r.meta = *reinterpret_cast<GLOBAL_AS const uint32_t*>(rec + 24 * L);
        return r;
    };
    // DEPTH records in flight per lane group (a pass of the block is one dependent chain spike id -> record -> adds, and a
    // step of a few thousand spikes is only a handful of passes per block): ids are fetched 2 * DEPTH passes ahead of their
    // adds, records DEPTH passes ahead.  Every value that is loaded keeps ONE place for the whole loop — id slot v, record
    // slot v % DEPTH, used up before it is loaded again, the round written out 2 * DEPTH passes long so that no id moves
    // from slot to slot: a loaded value that changes its register where the loop closes is copied there, and that copy
    // waits for every load issued before it, i.e. drains the pipeline once per round (the loop ran at a quarter of its
    // present speed that way).
    constexpr uint32_t DEPTH = 4;
    uint32_t s = G.split * perBlock + (threadIdx.x / WAVE) * GROUPS + min(group, GROUPS - 1);
    uint32_t ids[2 * DEPTH];
    Rec recs[DEPTH];
    // A segment longer than a record (one in seven where segments average 16 synapses, so nearly every pass of a
    // wavefront's twelve records holds one) has its next 8 synapses in an overflow record.  That record is asked for when
    // the segment's length is known and added DEPTH passes later, when the slot comes round again: read and added on the
    // spot, it cost every pass a whole trip to memory, and with it every load in flight was waited for.
    struct Ovf { float w0, w1; uint32_t t0, t1, m; };
    Ovf ovf[DEPTH];
    #pragma unroll
    for(uint32_t u = 0; u < DEPTH; u++) { ovf[u].w0 = ovf[u].w1 = 0.0f; ovf[u].t0 = ovf[u].t1 = 0u; ovf[u].m = 0u; }
    auto addOverflow = [&](Ovf &o) {
        if(o.m) {
            ldsAddF32x2(&shTile[o.t0], o.w0, k < o.m, &shTile[o.t1], o.w1, k + L < o.m);
            o.m = 0u;
        }
    };
    #pragma unroll
    for(uint32_t v = 0; v < 2 * DEPTH; v++) { ids[v] = spk[min(s + v * stride, lastSrc)]; }
    #pragma unroll
    for(uint32_t u = 0; u < DEPTH; u++) { recs[u] = fetch(ids[u]); }
    // (the loop is entered with no load pending: the waits inside it are then counted from the loop's own order of loads
    // alone; merged with this prologue's order they come out as "all but the last two or three" on every round)
    __builtin_amdgcn_s_waitcnt(0);
    for(; s < numSpikes; s += 2 * DEPTH * stride) {
        #pragma unroll
        for(uint32_t v = 0; v < 2 * DEPTH; v++) {
            Rec &cur = recs[v % DEPTH];
            Ovf &pend = ovf[v % DEPTH];
            addOverflow(pend);
            if(live && s + v * stride < numSpikes) {
                const uint32_t idPre = ids[v];
                const uint32_t n = cur.meta & 0xFFFFu;
                const uint32_t j = 4 * k;
                ldsAddF32x4(&shTile[cur.t01 & 0xFFFFu], cur.w.x, j < n, &shTile[cur.t01 >> 16], cur.w.y, j + 1 < n,
                            &shTile[cur.t23 & 0xFFFFu], cur.w.z, j + 2 < n, &shTile[cur.t23 >> 16], cur.w.w, j + 3 < n);
                if(n > C) {
                    uint32_t done = C;
                    if(overflow) {
                        GLOBAL_AS const uint8_t *rec = overflow + (size_t)idPre * 64;
                        const uint32_t m = min(n - C, REC_OVERFLOW);
                        if(k < m) { pend.w0 = reinterpret_cast<GLOBAL_AS const float*>(rec)[k]; pend.t0 = reinterpret_cast<GLOBAL_AS const uint16_t*>(rec + 32)[k]; }
                        if(k + L < m) { pend.w1 = reinterpret_cast<GLOBAL_AS const float*>(rec)[k + L]; pend.t1 = reinterpret_cast<GLOBAL_AS const uint16_t*>(rec + 32)[k + L]; }
                        pend.m = m;
                        done = C + REC_OVERFLOW;
                    }
                    if(n > done) {
                        // beyond both records (rare): from the row itself, on the spot
                        const size_t base = (size_t)idPre * g.rowStride + (cur.meta >> 16);
                        for(uint32_t jj = done + k; jj < n; jj += L) {
                            ldsAddF32(&shTile[asGlobal(g.ind)[base + jj] - tileStart], asGlobal(g.g)[base + jj]);
                        }
                    }
                }
                if(k == 0) { events += n; }
            }
            cur = fetch(ids[(v + DEPTH) % (2 * DEPTH)]);
            ids[v] = spk[min(s + (v + 2 * DEPTH) * stride, lastSrc)];
        }
    }
    #pragma unroll
    for(uint32_t u = 0; u < DEPTH; u++) { addOverflow(ovf[u]); }
    return events;
}

__device__ __forceinline__ void presynapticTileBody(const TileGroupDev &G, float *shTile, const StepArgs &args, float dt, unsigned long long *eventCounter)
{
    const gennmi_presynaptic_update_group_t &g = G.g;
    const uint32_t batch = blockIdx.y;
    const uint32_t numSpikes = asGlobal(g.srcSpkCnt)[batch];
    if((unsigned long long)numSpikes * g.rowStride < G.threshold) { return; }      // the scatter kernel took this step
    if(G.recLanes) {
        // A step with few spikes is shared between fewer blocks per tile: every block zeroes a whole tile and flushes what it
        // touched with global atomics, which costs more than the adds themselves while a block's share of the tile is
        // sparsely filled.  Measured on 10^6 rows x 1000 synapses (us per step with 2 / 4 / 8 / 16 blocks per tile): 3 x 10^3
        // spikes 49 / 54 / 73 / 102, 2 x 10^4 spikes 171 / 114 / 111 / 159, 3 x 10^5 spikes 2281 / 1190 / 754 / 766.
        const uint32_t activeSplits = min(G.numSplits, max(2u, numSpikes / G.spikesPerSplit));
        if(G.split >= activeSplits) { return; }
        const uint32_t tileStart = G.tile * G.tileSize;
        const uint32_t tileLen = min(G.tileSize, g.numTrgNeurons - tileStart);
        for(uint32_t k = threadIdx.x; k < tileLen; k += blockDim.x) { shTile[k] = 0.0f; }
        __syncthreads();
        GLOBAL_AS const uint32_t *spk = asGlobal(g.srcSpk) + (size_t)batch * g.numSrcNeurons;
        unsigned long long events = (G.recLanes == 5) ? tileRecordLoop<5>(G, spk, numSpikes, activeSplits, shTile, tileStart)
                                                      : tileRecordLoop<10>(G, spk, numSpikes, activeSplits, shTile, tileStart);
        __syncthreads();
        GLOBAL_AS float *outPost = asGlobal(g.outPost) + (size_t)batch * g.numTrgNeurons + tileStart;
        for(uint32_t k = threadIdx.x; k < tileLen; k += blockDim.x) {
            const float v = shTile[k];
            if(v != 0.0f) { atomicAddF32(&outPost[k], v); }
        }
        for(int o2 = WAVE / 2; o2 > 0; o2 >>= 1) { events += __shfl_down(events, o2, WAVE); }
        if((threadIdx.x & (WAVE - 1)) == 0 && events) { addEvents(eventCounter, events); }
        return;
    }
    const uint32_t tileStart = G.tile * G.tileSize;
    const uint32_t tileLen = min(G.tileSize, g.numTrgNeurons - tileStart);
    for(uint32_t k = threadIdx.x; k < tileLen; k += blockDim.x) { shTile[k] = 0.0f; }
    __syncthreads();

    GLOBAL_AS const uint32_t *spk = asGlobal(g.srcSpk) + (size_t)batch * g.numSrcNeurons;
    GLOBAL_AS const uint16_t *off = asGlobal(G.tileOff);
    GLOBAL_AS const uint32_t *ind = asGlobal(g.ind);
    // trace-STDP rows: besides delivering the (old) weight, every event applies the presynaptic-spike rule to its own
    // synapse (pygenn/genn_model.py:1456-1463); a synapse belongs to exactly one tile, so g needs no atomic here either.
    // Plastic weights, spike times and traces are per batch.
    const bool additive = (g.wum == GENNMI_WUM_STDP);
    const bool stdp = (g.wum == GENNMI_WUM_STDP_TRACE) || additive;
    GLOBAL_AS float *weight = asGlobal(g.g) + (stdp ? (size_t)batch * g.numSrcNeurons * g.rowStride : (size_t)0);
    const float t = stdp ? resolve(args, dt).t : 0.0f;
    GLOBAL_AS const float *trgST = asGlobal(g.trgST) + (size_t)batch * g.numTrgNeurons;
    GLOBAL_AS const float *postTrace = asGlobal(g.postTrace) + (size_t)batch * g.numTrgNeurons;
    GLOBAL_AS const uint32_t *trgBitmap = asGlobal(G.learn.trgBitmap) + (size_t)batch * ((g.numTrgNeurons + 31) / 32);
    const bool paired = (G.learn.enabled != 0);
    // the rule on one synapse, given what it reads of its target: last spike time, trace, word of the spike bitmap
    // (what the postsynaptic-spike rule reads of the row's own neuron — rowST, rowTrace — is loaded once per row, one row ahead:
    // in a burst most targets have just fired, and two dependent loads per synapse were the longest chain of such a step)
    float rowST = 0.0f, rowTrace = 0.0f;
    auto depressWith = [&](uint32_t idPre, uint32_t idPost, float w, float st, float trace, uint32_t bits) -> float {
        const float stPost = dt + st;
        const float dtSpike = t - stPost;
        float nw = w;
        if(dtSpike > 0) {
            const float factor = additive ? (float)exp((double)(-dtSpike / g.tauMinus)) : trace;
            nw = fminf(g.wMax, fmaxf(g.wMin, w - (g.aMinus * factor)));
        }
        // the target fired in the last update too: its postsynaptic-spike rule follows here (see LearnPostDev)
        if(paired && ((bits >> (idPost & 31u)) & 1u)) { nw = learnPostOnSynapseWith(G.learn, g, rowST, rowTrace, nw, t, dt); }
        return nw;
    };
    auto depress = [&](uint32_t idPre, uint32_t idPost, float w) -> float {
        return depressWith(idPre, idPost, w, trgST[idPost], additive ? 0.0f : postTrace[idPost], paired ? trgBitmap[idPost >> 5] : 0u);
    };
    // four synapses of a lane: all their gathers are issued before the first is used (one synapse at a time, each waits
    // for its own two or three dependent loads: twelve trips to L2 in a row per lane and pass)
    auto depress4 = [&](uint32_t idPre, const u32x4u &ip, const f32x4u &w) -> f32x4u {
        const float st0 = trgST[ip.x], st1 = trgST[ip.y], st2 = trgST[ip.z], st3 = trgST[ip.w];
        float tr0 = 0.0f, tr1 = 0.0f, tr2 = 0.0f, tr3 = 0.0f;
        if(!additive) { tr0 = postTrace[ip.x]; tr1 = postTrace[ip.y]; tr2 = postTrace[ip.z]; tr3 = postTrace[ip.w]; }
        uint32_t b0 = 0, b1 = 0, b2 = 0, b3 = 0;
        if(paired) { b0 = trgBitmap[ip.x >> 5]; b1 = trgBitmap[ip.y >> 5]; b2 = trgBitmap[ip.z >> 5]; b3 = trgBitmap[ip.w >> 5]; }
        f32x4u nw;
        nw.x = depressWith(idPre, ip.x, w.x, st0, tr0, b0); nw.y = depressWith(idPre, ip.y, w.y, st1, tr1, b1);
        nw.z = depressWith(idPre, ip.z, w.z, st2, tr2, b2); nw.w = depressWith(idPre, ip.w, w.w, st3, tr3, b3);
        return nw;
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
    GLOBAL_AS const float *srcST = asGlobal(G.learn.srcST) + (size_t)batch * g.numSrcNeurons;
    GLOBAL_AS const float *preTrace = asGlobal(G.learn.preTrace) + (size_t)batch * g.numSrcNeurons;
    const bool rowTraceWanted = paired && !(G.learn.tauPlus > 0.0f);
    float st0 = paired ? srcST[id0] : 0.0f, tr0 = rowTraceWanted ? preTrace[id0] : 0.0f;
    for(; s < numSpikes; s += stride) {
        const uint32_t idPre = id0, a = a0, b = b0;
        rowST = st0; rowTrace = tr0;
        id0 = id1;
        id1 = spk[min(s + 2 * stride, lastSrc)];
        o0 = (size_t)id0 * (G.numTiles + 1) + G.tile;
        a0 = off[o0]; b0 = off[o0 + 1];
        if(paired) { st0 = srcST[id0]; }
        if(rowTraceWanted) { tr0 = preTrace[id0]; }
        const size_t rowBase = (size_t)idPre * g.rowStride;
        for(uint32_t j = a + 4 * lis; j < b; j += 4 * L) {
            if(j + 4 <= b) {
                const u32x4u ip = *reinterpret_cast<GLOBAL_AS const u32x4u*>(ind + rowBase + j);
                const f32x4u w = *reinterpret_cast<GLOBAL_AS const f32x4u*>(weight + rowBase + j);
                if(stdp) { *reinterpret_cast<GLOBAL_AS f32x4u*>(weight + rowBase + j) = depress4(idPre, ip, w); }
                ldsAddF32x4(&shTile[ip.x - tileStart], w.x, true, &shTile[ip.y - tileStart], w.y, true,
                            &shTile[ip.z - tileStart], w.z, true, &shTile[ip.w - tileStart], w.w, true);
            }
            else {
                for(uint32_t jj = j; jj < b; jj++) {
                    const uint32_t idPost = ind[rowBase + jj];
                    const float w = weight[rowBase + jj];
                    if(stdp) { weight[rowBase + jj] = depress(idPre, idPost, w); }
                    ldsAddF32(&shTile[idPost - tileStart], w);
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
    if((threadIdx.x & (WAVE - 1)) == 0 && events) { addEvents(eventCounter, events); }
}

__global__ __launch_bounds__(1024)
void presynapticTileKernel(const TileGroupDev * __restrict__ blocks, StepArgs args, float dt, unsigned long long *eventCounter)
{
    extern __shared__ float shTile[];
    presynapticTileBody(blocks[blockIdx.x], shTile, args, dt, eventCounter);
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
    if(lane == 0 && events) { addEvents(eventCounter, events); }
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

// Builds the segment records of one projection from its rows and the segment boundaries: one thread per (tile, row).
template<uint32_t L>
__global__ __launch_bounds__(BLOCK)
void tileRecordBuildKernel(uint32_t numSrc, uint32_t rowStride, const uint32_t *ind, const float *weight, const uint16_t *off,
                           uint32_t tileSize, uint32_t numTiles, uint8_t *records, uint8_t *overflow)
{
    constexpr uint32_t C = 4 * L, REC = recordBytes(L);
    const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if(idx >= (size_t)numSrc * numTiles) { return; }
    const uint32_t tile = (uint32_t)(idx / numSrc), row = (uint32_t)(idx % numSrc);
    const uint32_t a = off[(size_t)row * (numTiles + 1) + tile], b = off[(size_t)row * (numTiles + 1) + tile + 1];
    const uint32_t n = b - a, tileStart = tile * tileSize;
    uint8_t *rec = records + idx * REC;
    const size_t base = (size_t)row * rowStride + a;
    for(uint32_t q = 0; q < L; q++) {
        f32x4 w; uint32_t t[4];
        for(uint32_t e = 0; e < 4; e++) {
            const uint32_t j = 4 * q + e;
            const bool valid = j < n;           // j < C always
            ((float*)&w)[e] = valid ? weight[base + j] : 0.0f;
            t[e] = valid ? (ind[base + j] - tileStart) : 0u;
        }
        *reinterpret_cast<f32x4*>(rec + 16 * q) = w;
        *reinterpret_cast<u32x2*>(rec + 16 * L + 8 * q) = u32x2{t[0] | (t[1] << 16), t[2] | (t[3] << 16)};
    }
    *reinterpret_cast<u32x2*>(rec + 24 * L) = u32x2{n | (a << 16), 0u};
    if(overflow && n > C) {
        uint8_t *ovf = overflow + idx * 64;
        for(uint32_t e = 0; e < REC_OVERFLOW; e++) {
            const bool valid = C + e < n;
            reinterpret_cast<float*>(ovf)[e] = valid ? weight[base + C + e] : 0.0f;
            reinterpret_cast<uint16_t*>(ovf + 32)[e] = valid ? (uint16_t)(ind[base + C + e] - tileStart) : (uint16_t)0;
        }
    }
}

// ------------------------------------------------------------------------------------------------
// Toeplitz Conv2D on the matrix cores (fp32 MFMA: products of a 0 / 1 spike indicator and an fp32 weight are exact, the
// sums are fp32 like every other path's; only their order differs from the CPU backend's queue order).
//
//   outPost[y][x][o] += sum over (a, b, ch) of S[y + a - PH][x + b - PW][ch] * kernel[a][b][ch][o],
//   PH = kh - 1 - convBH, PW = kw - 1 - convBW
// is the gather form of initToeplitzConnectivitySnippet.h:116-137 (a, b are the kernel taps counted from the far corner).
// A block owns `rowsPerBlock` output rows of one batch.  It expands the bits of the input rows those reach into a planar
// patch in LDS ([channel][row][column], so that the 32 pixels of an MFMA tile read consecutive words), copies the kernel
// next to it, and every wavefront then computes tiles of 32 pixels x 32 output channels with v_mfma_f32_32x32x2_f32, two
// steps of the (tap, channel) sum per instruction, and adds its tile to outPost (the block owns these rows).
// ------------------------------------------------------------------------------------------------
constexpr int CONV_MFMA_THREADS = 512;       // eight wavefronts: a compute unit then holds one block, whose wavefronts start together
constexpr int CONV_MFMA_STEPS = 72;         // steps of the (tap, channel) sum per unrolled chunk of the inner loop
constexpr int CONV_MFMA_AHEAD = 6;          // steps whose operands are fetched ahead of the matrix instructions (divides the above)

// what a block does with a finished tile of 32 pixels x 32 output channels: here, add it to outPost
struct ConvAddToOutPost
{
    GLOBAL_AS float *outPost;           // of this batch
    uint32_t ow, oc;
    __device__ __forceinline__ void prefetch(uint32_t, uint32_t, uint32_t, uint32_t, uint32_t) {}
    __device__ __forceinline__ void finish(const f32x16 &acc, uint32_t, uint32_t y, uint32_t x0, uint32_t o, uint32_t half)
    {
        // one atomic without return per element and step, so the result does not depend on their order (a read-modify-write
        // by the owning lane measured no faster)
        #pragma unroll
        for(int v = 0; v < 16; v++) {
            const uint32_t x = x0 + 8 * (v / 4) + 4 * half + (v % 4);
            if(x < ow && o < oc && acc[v] != 0.0f) { atomicAddF32(&outPost[((size_t)y * ow + x) * oc + o], acc[v]); }
        }
    }
};

// floats of LDS that a block's input patch and its copy of the kernel take (what follows them belongs to the caller)
__device__ __forceinline__ uint32_t convMfmaLdsFloats(const ConvMfmaDev &G)
{
    const uint32_t K = (uint32_t)(G.g.conv[0] * G.g.conv[1] * G.g.conv[4]), steps = (K + 1) / 2;
    return (uint32_t)G.g.conv[4] * G.planePitch + 2 * ((steps + CONV_MFMA_STEPS - 1) / CONV_MFMA_STEPS) * CONV_MFMA_STEPS * G.kernPitch;
}

// the output rows [rowGroup * rowsPerBlock, ...) of one batch, by all THREADS threads of a block; `epoch`: completed steps
template<int THREADS, typename Epilogue>
__device__ __forceinline__ void convMfmaBlock(const ConvMfmaDev &G, uint32_t rowGroup, uint32_t batch, unsigned long long epoch, float *lds,
                                              Epilogue &epilogue, unsigned long long *eventCounter, unsigned long long *waveEvents = nullptr)
{
    const gennmi_presynaptic_update_group_t &g = G.g;
    const int kh = g.conv[0], kw = g.conv[1], ih = g.conv[2], iw = g.conv[3], ic = g.conv[4];
    const int oh = g.conv[5], ow = g.conv[6], oc = g.conv[7];
    const uint32_t planePitch = G.planePitch, patchPitch = G.patchPitch, kernPitch = G.kernPitch;
    const int y0 = (int)(rowGroup * G.rowsPerBlock);
    const int rows = min((int)G.rowsPerBlock, oh - y0);
    const int PH = kh - 1 - G.convBH, PW = kw - 1 - G.convBW;
    const uint32_t K = (uint32_t)(kh * kw * ic), steps = (K + 1) / 2;
    // kernel rows in LDS: whole chunks of steps, so that the unrolled loop needs no guard (rows beyond K are zero)
    const uint32_t kernRows = 2 * ((steps + CONV_MFMA_STEPS - 1) / CONV_MFMA_STEPS) * CONV_MFMA_STEPS;
    float *patch = lds;
    float *kern = patch + (size_t)ic * planePitch;
    const uint32_t lane = threadIdx.x & (WAVE - 1), wave = threadIdx.x / WAVE;
    const uint32_t half = lane >> 5, col = lane & 31;
    GLOBAL_AS const uint32_t *bitmap = asGlobal(G.srcBitmap) + (epoch & 1) * G.bitmapStride + (size_t)batch * ((g.numSrcNeurons + 31) / 32);
    GLOBAL_AS const float *kernel = asGlobal(g.g);
    const uint32_t xTiles = ((uint32_t)ow + 31) / 32, oTiles = ((uint32_t)oc + 31) / 32;
    const uint32_t numTiles = (uint32_t)rows * xTiles * oTiles;

    // ---- requested before anything is waited for: what the epilogue wants of the wavefront's first tile, this thread's first
    // words of the bitmap, the kernel
    if(wave < numTiles) {
        const uint32_t r = wave / (xTiles * oTiles), x0 = ((wave / oTiles) % xTiles) * 32, n0 = (wave % oTiles) * 32;
        epilogue.prefetch(r, (uint32_t)y0 + r, x0, n0 + col, half);
    }
    const int patchRows = rows + kh - 1;
    const uint32_t patchElems = (uint32_t)patchRows * patchPitch;
    auto pixelOf = [&](uint32_t e, int &inRow, int &inCol) -> bool {
        const int r = (int)(e / patchPitch), c = (int)(e - (uint32_t)r * patchPitch);
        inRow = y0 - PH + r; inCol = c - PW;
        return (e < patchElems && inRow >= 0 && inRow < ih && inCol >= 0 && inCol < iw);
    };
    // (a thread's first two pixels: all there is to do for patches of up to 2 x THREADS elements)
    int inRow0, inCol0, inRow1, inCol1;
    const bool inside0 = pixelOf(threadIdx.x, inRow0, inCol0), inside1 = pixelOf(threadIdx.x + THREADS, inRow1, inCol1);
    const uint32_t first0 = inside0 ? (uint32_t)((inRow0 * iw + inCol0) * ic) : 0u, first1 = inside1 ? (uint32_t)((inRow1 * iw + inCol1) * ic) : 0u;
    const uint32_t word0 = bitmap[first0 >> 5], word1 = bitmap[first1 >> 5];

    // ---- kernel weights [k][o] into LDS, rows padded to kernPitch
    if(kernPitch == (uint32_t)oc && (oc & 3) == 0 && (reinterpret_cast<uintptr_t>(g.g) & 15) == 0) {
        // rows are contiguous on both sides: 16 bytes per load, up to eight loads in flight per thread
        const uint32_t quads = K * (uint32_t)oc / 4, allQuads = kernRows * kernPitch / 4;
        GLOBAL_AS const f32x4 *src = reinterpret_cast<GLOBAL_AS const f32x4*>(kernel);
        f32x4 *dst = reinterpret_cast<f32x4*>(kern);
        for(uint32_t q0 = 0; q0 < allQuads; q0 += 8 * THREADS) {
            f32x4 w[8];
            #pragma unroll
            for(int u = 0; u < 8; u++) { const uint32_t q = q0 + u * THREADS + threadIdx.x; w[u] = src[min(q, quads - 1)]; }
            #pragma unroll
            for(int u = 0; u < 8; u++) {
                const uint32_t q = q0 + u * THREADS + threadIdx.x;
                const f32x4 zero = {0, 0, 0, 0};
                if(q < allQuads) { dst[q] = (q < quads) ? w[u] : zero; }
            }
        }
    }
    else {
        for(uint32_t e0 = 0; e0 < kernRows * kernPitch; e0 += 8 * THREADS) {
            float w[8];
            #pragma unroll
            for(int u = 0; u < 8; u++) {
                const uint32_t e = e0 + u * THREADS + threadIdx.x;
                const uint32_t k = e / kernPitch, o = e - k * kernPitch;
                w[u] = kernel[(size_t)min(k, K - 1) * oc + min(o, (uint32_t)oc - 1)] * ((k < K && o < (uint32_t)oc) ? 1.0f : 0.0f);
            }
            #pragma unroll
            for(int u = 0; u < 8; u++) {
                const uint32_t e = e0 + u * THREADS + threadIdx.x;
                if(e < kernRows * kernPitch) { kern[e] = w[u]; }
            }
        }
    }
    // ---- input patch: bit (row * iw + col) * ic + ch of the source's bitmap -> patch[ch][r][c].  A pixel's spikes are
    // counted as events by the block whose output rows include the pixel's row (the last block takes the rows below):
    // every spike reaches kh * kw * oc targets less what falls outside the output.
    unsigned long long events = 0;
    const bool lastBlock = (y0 + rows >= oh);
    for(uint32_t e = threadIdx.x; e < patchElems; e += THREADS) {
        int inRow, inCol;
        const bool inside = pixelOf(e, inRow, inCol);
        const uint32_t id0 = inside ? (uint32_t)((inRow * iw + inCol) * ic) : 0u;
        uint32_t wordIdx = id0 >> 5, word = (e == threadIdx.x) ? word0 : (e == threadIdx.x + THREADS) ? word1 : bitmap[wordIdx], fired = 0;
        for(int ch = 0; ch < ic; ch++) {
            const uint32_t id = id0 + (uint32_t)ch;
            if(inside && (id >> 5) != wordIdx) { wordIdx = id >> 5; word = bitmap[wordIdx]; }
            const bool bit = inside && ((word >> (id & 31)) & 1u);
            patch[(size_t)ch * planePitch + e] = bit ? 1.0f : 0.0f;
            fired += bit ? 1u : 0u;
        }
        if(fired && inRow >= y0 && (inRow < y0 + rows || lastBlock)) {
            int rowTaps = 0, colTaps = 0;
            for(int kr = 0; kr < kh; kr++) { const int pr = inRow + kr - G.convBH; rowTaps += (pr >= 0 && pr < oh) ? 1 : 0; }
            for(int kc = 0; kc < kw; kc++) { const int pc = inCol + kc - G.convBW; colTaps += (pc >= 0 && pc < ow) ? 1 : 0; }
            events += (unsigned long long)fired * (unsigned long long)(rowTaps * colTaps * oc);
        }
    }
    __syncthreads();

    // A[i][k]: pixel x0 + i, k = (a * kw + b) * ic + ch -> patch[ch][r + a][x0 + i + b];  B[k][j] = kern[k][n0 + j]; the
    // two halves of the wavefront take k = 2 s and 2 s + 1.  Where step s starts in the patch is worked out once per chunk
    // of steps, lane L keeping the offsets of steps L and L + 64 for either half; the loop fetches them with readlane, so
    // it holds no division and no branch and its LDS reads can all be in flight ahead of the matrix instructions.
    auto patchOffsetOf = [&](uint32_t k) -> uint32_t {
        const uint32_t kk = min(k, K - 1);                          // (beyond K: any valid place, B is zero there)
        const uint32_t tap = kk / (uint32_t)ic, ch = kk - tap * (uint32_t)ic;
        const uint32_t ta = tap / (uint32_t)kw;
        return ch * planePitch + ta * patchPitch + (tap - ta * (uint32_t)kw);
    };
    for(uint32_t tile = wave; tile < numTiles; tile += THREADS / WAVE) {
        const uint32_t r = tile / (xTiles * oTiles), x0 = ((tile / oTiles) % xTiles) * 32, n0 = (tile % oTiles) * 32;
        const uint32_t y = (uint32_t)y0 + r, o = n0 + col;
        f32x16 acc = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
        if(tile != wave) { epilogue.prefetch(r, y, x0, o, half); }
        const float *aBase = patch + r * patchPitch + x0 + col;
        for(uint32_t s0 = 0; s0 < steps; s0 += CONV_MFMA_STEPS) {
            const int evenLo = (int)patchOffsetOf(2 * (s0 + lane)), oddLo = (int)patchOffsetOf(2 * (s0 + lane) + 1);
            const int evenHi = (int)patchOffsetOf(2 * (s0 + lane + WAVE)), oddHi = (int)patchOffsetOf(2 * (s0 + lane + WAVE) + 1);
            const float *bBase = kern + (size_t)(2 * s0 + half) * kernPitch + n0 + col;
            // software pipeline: the operands of the next CONV_MFMA_AHEAD steps are read from LDS while the matrix
            // instructions of the current ones run (the scheduling barriers keep the reads where they are written: left to itself
            // the compiler sinks every read to just before its use)
            constexpr int AHEAD = CONV_MFMA_AHEAD;
            float av[2][AHEAD], bv[2][AHEAD];
            auto fetch = [&](int buffer, int first) {
                #pragma unroll
                for(int u = 0; u < AHEAD; u++) {
                    const int s = first + u;
                    const int even = __builtin_amdgcn_readlane((s < WAVE) ? evenLo : evenHi, s & (WAVE - 1));
                    const int odd = __builtin_amdgcn_readlane((s < WAVE) ? oddLo : oddHi, s & (WAVE - 1));
                    av[buffer][u] = aBase[half ? odd : even];
                    bv[buffer][u] = bBase[(size_t)2 * s * kernPitch];
                }
            };
            fetch(0, 0);
            #pragma unroll
            for(int c = 0; c < CONV_MFMA_STEPS / AHEAD; c++) {
                __builtin_amdgcn_sched_barrier(0);
                if(c + 1 < CONV_MFMA_STEPS / AHEAD) { fetch((c + 1) & 1, (c + 1) * AHEAD); }
                __builtin_amdgcn_sched_barrier(0);
                #pragma unroll
                for(int u = 0; u < AHEAD; u++) { acc = __builtin_amdgcn_mfma_f32_32x32x2f32(av[c & 1][u], bv[c & 1][u], acc, 0, 0, 0); }
            }
        }
        // register v of lane (half, col) holds D[i][j] with i = 8 * (v / 4) + 4 * half + v % 4, j = col: the 32 lanes of a
        // half hold the 32 consecutive channels of one pixel
        epilogue.finish(acc, r, y, x0, o, half);
    }
    for(int o2 = WAVE / 2; o2 > 0; o2 >>= 1) { events += __shfl_down(events, o2, WAVE); }
    // (a caller with barriers still to come takes the wavefronts' sums in LDS and adds them itself when it is done: a barrier
    // waits for the wavefront's memory operations, and a thousand atomics on the one counter complete one after the other)
    if(lane == 0) {
        if(waveEvents) { waveEvents[wave] = events; }
        else if(events) { addEvents(eventCounter, events); }
    }
}

__global__ __launch_bounds__(CONV_MFMA_THREADS)
void presynapticConvMfmaKernel(const ConvMfmaDev * __restrict__ blocks, uint32_t mfmaBlocks, const PreGroupDev * __restrict__ scatter,
                               StepArgs args, float dt, unsigned long long *eventCounter)
{
    extern __shared__ float shConvM[];
    const ConvMfmaDev &G = blocks[0];
    const gennmi_presynaptic_update_group_t &g = G.g;
    // Blocks are numbered batch-first (block = index * numBatches + batch), so that consecutive work-groups, which go to
    // consecutive XCDs, differ in batch.  Behind the blocks of the dense path come those of the scatter path, which takes
    // the steps too quiet for it: one launch, and the device decides which of the two does the work.
    const uint32_t numBatches = G.numBatches;
    const uint32_t batch = blockIdx.x % numBatches;
    const Resolved st = resolve(args, dt);
    if(blockIdx.x >= mfmaBlocks) {
        const uint32_t b = (blockIdx.x - mfmaBlocks) / numBatches;
        presynapticBody(scatter[b], b, batch, numBatches, st, dt, eventCounter);
        return;
    }
    const uint32_t numDiag = (uint32_t)(g.conv[0] * g.conv[1] * g.conv[7]);
    const uint32_t numSpikes = asGlobal(g.srcSpkCnt)[batch];
    if((unsigned long long)numSpikes * numDiag < G.threshold) { return; }      // the scatter kernel took this step
    ConvAddToOutPost epilogue{asGlobal(g.outPost) + (size_t)batch * g.numTrgNeurons, (uint32_t)g.conv[6], (uint32_t)g.conv[7]};
    convMfmaBlock<CONV_MFMA_THREADS>(G, blockIdx.x / numBatches, batch, st.epoch, shConvM, epilogue, eventCounter);
}

// bitmap of a population's spike queue, for callers that wrote the queue themselves (the neuron update keeps it otherwise)
__global__ void spikeBitmapFromQueueKernel(const uint32_t *spkCnt, const uint32_t *spk, uint32_t *bitmap, uint32_t numNeurons, uint32_t clear)
{
    const uint32_t batch = blockIdx.y, words = (numNeurons + 31) / 32;
    const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
    if(clear) { if(i < words) { bitmap[(size_t)batch * words + i] = 0u; } return; }
    if(i < spkCnt[batch]) { const uint32_t id = spk[(size_t)batch * numNeurons + i]; atomicOr(&bitmap[(size_t)batch * words + (id >> 5)], 1u << (id & 31)); }
}

__global__ __launch_bounds__(1024)
void presynapticUpdateKernel(const PreGroupDev * __restrict__ blocks, StepArgs args, float dt, unsigned long long *eventCounter)
{
    presynapticBody(blocks[blockIdx.x], blockIdx.x, blockIdx.y, gridDim.y, resolve(args, dt), dt, eventCounter);
}

// ------------------------------------------------------------------------------------------------
// Postsynaptic update (learnPost): one sub-group per postsynaptic spike walks the column through
// remap (coalesced), gathers g by synapse index.
// ------------------------------------------------------------------------------------------------
__device__ __forceinline__ void postsynapticBody(const PostGroupDev &G, uint32_t blockInKernel, uint32_t *shBits, const Resolved &st, float dt)
{
    const gennmi_postsynaptic_update_group_t &g = G.g;
    const uint32_t batch = blockIdx.y;
    const uint32_t BS = blockDim.x;
    const uint32_t W = G.lanesPerSpike;
    const uint32_t localBlock = blockInKernel - G.startBlock;
    const uint32_t lis = threadIdx.x & (W - 1);
    // Sub-groups are numbered across the blocks first (sub-group k of block b is number k * numBlocks + b): a column walk is
    // a stream of scattered accesses, which a compute unit issues at one lane per clock, so the first spikes of the queue
    // should each find a compute unit of their own rather than share the first block's.
    const uint32_t subGroup = (threadIdx.x / W) * G.numBlocks + localBlock;
    const uint32_t numSubGroups = (G.numBlocks * BS) / W;
    // plastic weights, spike times and traces are per batch (VarAccess::READ_WRITE variables are duplicated); connectivity is shared
    const uint32_t numSpikes = g.trgSpkCnt[batch];
    GLOBAL_AS const uint32_t *trgSpk = asGlobal(g.trgSpk) + (size_t)batch * g.numTrgNeurons;
    GLOBAL_AS float *weight = asGlobal(g.g) + (size_t)batch * g.numSrcNeurons * g.rowStride;
    GLOBAL_AS const float *srcST = asGlobal(g.srcST) + (size_t)batch * g.numSrcNeurons;
    GLOBAL_AS const float *preTrace = asGlobal(g.preTrace) + (size_t)batch * g.numSrcNeurons;
    // rows of neurons that fired in the last update are left to the presynaptic pass, which applies this rule after its own
    GLOBAL_AS const uint32_t *srcBitmap = asGlobal(G.srcBitmap) + (size_t)batch * ((g.numSrcNeurons + 31) / 32);
    const bool paired = (G.srcBitmap != nullptr);
    const bool additive = (g.tauPlus > 0.0f);          // built-in rule (weightUpdateModels.h:360-366): no trace array
    if(G.denseThreshold && numSpikes >= G.denseThreshold) {
        // A large share of the target population fired: nearly every row holds synapses to update, so walk the rows
        // once (coalesced ind / g) and test each synapse's target against the spike bitmap, instead of one scattered
        // read-modify-write per (spike, column entry).  Same arithmetic per synapse; every synapse is visited once.
        const uint32_t words = (g.numTrgNeurons + 31) / 32;
        for(uint32_t k = threadIdx.x; k < words; k += BS) { shBits[k] = asGlobal(G.spikeBitmap)[(size_t)batch * words + k]; }
        __syncthreads();
        const uint32_t lane = threadIdx.x & (WAVE - 1);
        const uint32_t numWaves = G.numBlocks * (BS / WAVE);
        GLOBAL_AS const uint32_t *ind = asGlobal(g.ind);
        // per-row scalars of the NEXT row are fetched while the current one is processed (indices clamped: readable)
        const uint32_t lastRow = g.numSrcNeurons - 1;
        uint32_t row = localBlock * (BS / WAVE) + threadIdx.x / WAVE;
        uint32_t lenNext = asGlobal(g.rowLength)[min(row, lastRow)];
        float stNext = srcST[min(row, lastRow)], traceNext = additive ? 0.0f : preTrace[min(row, lastRow)];
        for(; row < g.numSrcNeurons; row += numWaves) {
            const uint32_t len = lenNext;
            const float stPre = dt + stNext;
            const float trace = traceNext;
            const uint32_t nextRow = min(row + numWaves, lastRow);
            lenNext = asGlobal(g.rowLength)[nextRow]; stNext = srcST[nextRow];
            if(!additive) { traceNext = preTrace[nextRow]; }
            const float dtSpike = st.t - stPre;
            if(!(dtSpike > 0) || len == 0 || (paired && bitmapTest(srcBitmap, row))) { continue; }
            const float step = g.aPlus * (additive ? (float)exp((double)(-dtSpike / g.tauPlus)) : trace);
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
    // A column entry is a chain of dependent memory round trips (remap -> spike time, trace and weight of that synapse ->
    // store), and a sub-group walks its column alone: four entries per lane are in flight at a time.  Every synapse is still
    // visited once, with the same arithmetic.
    constexpr int INFLIGHT = 4;
    GLOBAL_AS const uint32_t *remap = asGlobal(g.remap);
    for(uint32_t s = subGroup; s < numSpikes; s += numSubGroups) {
        const uint32_t spike = trgSpk[s];
        const uint32_t npre = asGlobal(g.colLength)[spike];
        const size_t colBase = (size_t)spike * g.colStride;
        for(uint32_t i0 = lis; i0 < npre; i0 += INFLIGHT * W) {
            uint32_t rowMajorIndex[INFLIGHT];
            bool live[INFLIGHT];
            #pragma unroll
            for(int u = 0; u < INFLIGHT; u++) {
                const uint32_t i = i0 + u * W;
                live[u] = (i < npre);
                rowMajorIndex[u] = live[u] ? remap[colBase + i] : 0u;
            }
            // second trip: everything an entry needs, for all four entries at once and whether the entry is live or not (a
            // dead one reads row 0 and synapse 0: readable) — loads that wait for the bitmap's answer, or sit behind a
            // branch per entry, are issued one entry after the other and the walk becomes nine trips long instead of three
            float stPre[INFLIGHT], trace[INFLIGHT], w[INFLIGHT];
            uint32_t firedBits[INFLIGHT], idPre[INFLIGHT];
            #pragma unroll
            for(int u = 0; u < INFLIGHT; u++) {
                idPre[u] = rowMajorIndex[u] / g.rowStride;
                firedBits[u] = paired ? srcBitmap[idPre[u] >> 5] : 0u;
                stPre[u] = srcST[idPre[u]];
                trace[u] = additive ? 0.0f : preTrace[idPre[u]];
                w[u] = weight[rowMajorIndex[u]];
            }
            #pragma unroll
            for(int u = 0; u < INFLIGHT; u++) { live[u] = live[u] && !((firedBits[u] >> (idPre[u] & 31u)) & 1u); }
            #pragma unroll
            for(int u = 0; u < INFLIGHT; u++) {
                const float dtSpike = st.t - (dt + stPre[u]);
                if(live[u] && dtSpike > 0) {
                    const float factor = additive ? (float)exp((double)(-dtSpike / g.tauPlus)) : trace[u];
                    const float newWeight = w[u] + (g.aPlus * factor);
                    weight[rowMajorIndex[u]] = fminf(g.wMax, fmaxf(g.wMin, newWeight));
                }
            }
        }
    }
}

__global__ __launch_bounds__(1024)
void postsynapticUpdateKernel(const PostGroupDev * __restrict__ blocks, StepArgs args, float dt)
{
    extern __shared__ uint32_t shBits[];
    postsynapticBody(blocks[blockIdx.x], blockIdx.x, shBits, resolve(args, dt), dt);
}

// All synaptic work of a step that can share a launch: the scatter path of every projection, the tile path of those that
// have one (a projection's step is taken by one or the other, decided on the device from its spike count) and the
// postsynaptic passes whose projections are paired with their presynaptic halves (LearnPostDev: no synapse is written by
// both, so nothing orders the passes).  Block ranges [0, preBlocks), [preBlocks, preBlocks + tileBlocks), then the rest.
__global__ __launch_bounds__(1024)
void synapseCombinedKernel(const PreGroupDev * __restrict__ pre, uint32_t preBlocks, const TileGroupDev * __restrict__ tiles, uint32_t tileBlocks,
                           const PostGroupDev * __restrict__ post, StepArgs args, float dt, unsigned long long *eventCounter)
{
    extern __shared__ float shDynamic[];
    if(blockIdx.x < preBlocks) {
        presynapticBody(pre[blockIdx.x], blockIdx.x, blockIdx.y, gridDim.y, resolve(args, dt), dt, eventCounter);
    }
    else if(blockIdx.x < preBlocks + tileBlocks) {
        presynapticTileBody(tiles[blockIdx.x - preBlocks], shDynamic, args, dt, eventCounter);
    }
    else {
        const uint32_t b = blockIdx.x - preBlocks - tileBlocks;
        postsynapticBody(post[b], b, reinterpret_cast<uint32_t*>(shDynamic), resolve(args, dt), dt);
    }
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
    if(len < 2 || len > REMAP_SORT_MAX) { return; }         // (longer columns: remapSortLongKernel)
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

// Columns too long for the LDS: the same kind of network in place, in global memory (a column of 10^5 entries stays in the
// L2), one work-group per column.  Every comparator of this form of the bitonic network puts the smaller entry at the
// lower index (a merge's first step pairs k with its mirror image in the block, k ^ (size - 1), the following ones k with
// k ^ stride), so positions beyond the column's length behave like entries of infinite value without being stored:
// a comparator that reaches beyond the length never exchanges.  (The reference's remap build has no limit on the column
// length, backendSIMT.cc:1977-1991.)
__global__ __launch_bounds__(BLOCK)
void remapSortLongKernel(uint32_t colStride, const uint32_t *colLength, uint32_t *remap)
{
    const uint32_t col = blockIdx.x;
    const uint32_t len = min(colLength[col], colStride);
    if(len <= REMAP_SORT_MAX) { return; }
    uint32_t p2 = 1;
    while(p2 < len) { p2 <<= 1; }
    uint32_t *column = remap + (size_t)col * colStride;
    for(uint32_t size = 2; size <= p2; size <<= 1) {
        for(uint32_t stride = size >> 1; stride > 0; stride >>= 1) {
            const uint32_t mask = (stride == (size >> 1)) ? size - 1u : stride;
            for(uint32_t k = threadIdx.x; k < len; k += BLOCK) {
                const uint32_t partner = k ^ mask;
                if(partner > k && partner < len) {
                    const uint32_t a = column[k], b = column[partner];
                    if(a > b) { column[k] = b; column[partner] = a; }
                }
            }
            __threadfence_block();
            __syncthreads();
        }
    }
}

uint32_t pow2Floor(uint32_t v) { uint32_t p = 1; while(p * 2 <= v) { p *= 2; } return p; }
uint32_t pow2Ceil(uint32_t v) { uint32_t p = 1; while(p < v) { p *= 2; } return p; }
}   // namespace

#endif
