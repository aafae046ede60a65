// Part of libgenn_mi355x.so: included by genn_mi355x.hip only (one translation unit).
//
// Ordered accumulation: a validation mode of the presynaptic update in which every postsynaptic element receives its
// synaptic input in exactly the order the reference's SingleThreadedCPU backend adds it
// (src/genn/backends/single_threaded_cpu/backend.cc:1884-1929: projections one after another, within a projection the
// spikes in queue order, within a spike's row the synapses in ascending position) — no atomics, one owner per element.
// The default kernels add the same values with fp32 atomics in whatever order the hardware retires them; this mode
// exists to show that nothing but that order separates their results from the CPU backend's.
//
// A projection is gathered through a column view of its matrix (for every postsynaptic neuron the synapse indices that
// target it, ascending — the order of the reference's own column build, backend.cc:156-179).  The spike queue is in
// ascending neuron index, so "queue order, then row order" is "ascending synapse index": a wavefront that owns one
// postsynaptic neuron walks its column 64 entries at a time, tests each entry's presynaptic neuron against a bitmap of
// the step's spikes, and adds the weights of the entries that fired one after another, in column order.
#ifndef GENN_MI355X_ORDERED_KERNELS_H
#define GENN_MI355X_ORDERED_KERNELS_H

namespace
{
constexpr uint32_t ORDERED_MAX_SLOT_REGS = 4;       // dendritic-delay rings of up to 256 slots (one accumulator per slot, 64 slots per register)

// one spike queue as a projection reads it (delay slot included): its spikes become a bitmap, once per step
struct OrderedSourceDev
{
    const uint32_t *srcSpkCnt, *srcSpk;
    uint32_t *bitmap;                   // [batch * words]
    uint32_t numSrcNeurons, words;
    uint32_t numSrcDelaySlots, axonalDelaySteps;
    uint32_t startBlock, numBlocks;
};

struct OrderedGroupDev
{
    gennmi_presynaptic_update_group_t g;
    const uint32_t *colLength;          // [numTrg]
    const uint32_t *remap;              // [numTrg * colStride] synapse indices of every column, ascending
    const uint32_t *bitmap;             // the source queue's bitmap of this step
    uint32_t colStride, words;
};

__global__ void orderedClearKernel(uint32_t *words, size_t count)
{
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if(i < count) { words[i] = 0u; }
}

__global__ __launch_bounds__(BLOCK)
void orderedBitmapKernel(const OrderedSourceDev * __restrict__ blocks, StepArgs args, float dt)
{
    const OrderedSourceDev &S = blocks[blockIdx.x];
    const Resolved st = resolve(args, dt);
    const uint32_t batch = blockIdx.y;
    const uint32_t slots = max(1u, S.numSrcDelaySlots);
    // the slot a projection with this axonal delay reads (backendBase.cc:207-216), as in the scatter kernel
    const uint32_t readSlot = (slots > 1) ? modStep(st.epoch + slots - S.axonalDelaySteps, slots) : 0u;
    const uint32_t count = S.srcSpkCnt[(size_t)batch * slots + readSlot];
    const uint32_t *spk = S.srcSpk + ((size_t)batch * slots + readSlot) * S.numSrcNeurons;
    uint32_t *bitmap = S.bitmap + (size_t)batch * S.words;
    for(uint32_t s = (blockIdx.x - S.startBlock) * BLOCK + threadIdx.x; s < count; s += S.numBlocks * BLOCK) {
        const uint32_t id = spk[s];
        atomicOr(&bitmap[id >> 5], 1u << (id & 31));
    }
}

// One wavefront per postsynaptic neuron; grid.y = batch.
__global__ __launch_bounds__(BLOCK)
void presynapticOrderedKernel(OrderedGroupDev G, StepArgs args, float dt, unsigned long long *eventCounter)
{
    const gennmi_presynaptic_update_group_t &g = G.g;
    const Resolved st = resolve(args, dt);
    const uint32_t lane = threadIdx.x & (WAVE - 1);
    const uint32_t idPost = blockIdx.x * (BLOCK / WAVE) + threadIdx.x / WAVE;
    if(idPost >= g.numTrgNeurons) { return; }
    const uint32_t batch = blockIdx.y;
    const uint32_t *bitmap = G.bitmap + (size_t)batch * G.words;
    const uint32_t D = g.maxDenDelay;
    const uint32_t denPtr = D ? modStep(st.epoch + 1, D) : 0u;      // the pointer in force during this step's synapse update
    float *outPost = g.outPost + (size_t)batch * g.numTrgNeurons;
    float *denDelay = D ? g.denDelay + (size_t)batch * D * g.numTrgNeurons : nullptr;
    const bool additive = (g.wum == GENNMI_WUM_STDP);
    const bool stdp = (g.wum == GENNMI_WUM_STDP_TRACE) || additive;

    // accumulators: the element itself (no ring), or one per ring slot, lane L of register q holding slot 64 q + L
    float acc[ORDERED_MAX_SLOT_REGS];
    #pragma unroll
    for(uint32_t q = 0; q < ORDERED_MAX_SLOT_REGS; q++) { acc[q] = 0.0f; }
    if(D == 0) { acc[0] = outPost[idPost]; }
    else {
        #pragma unroll
        for(uint32_t q = 0; q < ORDERED_MAX_SLOT_REGS; q++) {
            const uint32_t slot = q * WAVE + lane;
            if(slot < D) { acc[q] = denDelay[(size_t)slot * g.numTrgNeurons + idPost]; }
        }
    }
    // what the plastic rules read of the target neuron (same for every synapse of the column)
    float stPost = 0.0f, postTrace = 0.0f;
    if(stdp) {
        stPost = dt + g.trgST[idPost];          // st_post = DT * (backPropSteps + 1) + trgST  (synapseUpdateGroupMerged.cc:134-142)
        if(!additive) { postTrace = g.postTrace[idPost]; }
    }

    const uint32_t len = min(G.colLength[idPost], G.colStride);
    const uint32_t *column = G.remap + (size_t)idPost * G.colStride;
    unsigned long long events = 0;
    for(uint32_t base = 0; base < len; base += WAVE) {
        const uint32_t k = base + lane;
        const uint32_t idSyn = (k < len) ? column[k] : 0u;
        const uint32_t idPre = idSyn / g.rowStride;
        const bool active = (k < len) && ((bitmap[idPre >> 5] >> (idPre & 31)) & 1u);
        float w = 0.0f;
        uint32_t dl = 0u;
        if(active) {
            w = g.g[idSyn];
            if(D) { dl = g.d[idSyn]; }
            if(stdp) {
                // presynaptic-spike rule on the synapse this lane holds (pygenn/genn_model.py:1456-1463,
                // weightUpdateModels.h:352-359): the old weight is delivered, the new one stored
                const float dtSpike = st.t - stPost;
                if(dtSpike > 0) {
                    const float factor = additive ? (float)exp((double)(-dtSpike / g.tauMinus)) : postTrace;
                    g.g[idSyn] = fminf(g.wMax, fmaxf(g.wMin, w - (g.aMinus * factor)));
                }
            }
        }
        unsigned long long pending = __ballot(active);
        events += (unsigned long long)__popcll(pending);
        while(pending) {
            const int src = __ffsll((long long)pending) - 1;
            pending &= pending - 1;
            const float wv = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, w), src));
            if(D == 0) { acc[0] += wv; }
            else {
                const uint32_t slot = (denPtr + (uint32_t)__builtin_amdgcn_readlane((int)dl, src)) % D;
                #pragma unroll
                for(uint32_t q = 0; q < ORDERED_MAX_SLOT_REGS; q++) {
                    if(slot == q * WAVE + lane) { acc[q] += wv; }
                }
            }
        }
    }
    if(D == 0) { if(lane == 0) { outPost[idPost] = acc[0]; } }
    else {
        #pragma unroll
        for(uint32_t q = 0; q < ORDERED_MAX_SLOT_REGS; q++) {
            const uint32_t slot = q * WAVE + lane;
            if(slot < D) { denDelay[(size_t)slot * g.numTrgNeurons + idPost] = acc[q]; }
        }
    }
    if(lane == 0 && events) { addEvents(eventCounter, events); }
}
}   // namespace

#endif
