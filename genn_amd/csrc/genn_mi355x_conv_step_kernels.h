// A whole timestep of a convolutional layer in ONE launch (included by genn_mi355x.hip after the synapse and neuron kernels).
//
// The reference runs a Toeplitz Conv2D projection as updatePresynapticKernel (presynapticUpdateStrategySIMT.cc:750-934:
// one atomicAdd into outPost per (spike, kernel diagonal)) followed by updateNeuronsKernel (backendSIMT.cc:405-662), which
// reads outPost back.  On the matrix cores the layer's input of a step is a GEMM whose result a work-group holds in
// registers for whole output rows of one batch, so the postsynaptic model, the neuron model and the ordered spike queue can
// be applied to the accumulators where they are: `outPost` is read and written once like the rest of the neuron's state
// instead of receiving 2 million atomic adds that the neuron update then reads again, and the step is one launch.
//
// Grid (one-dimensional): the layer's work-groups (rowGroups x batches) first, then those of every other population (the
// layer's source).  A layer work-group owns `rowsPerBlock` output rows: it computes their input sums (convMfmaBlock), then per
// accumulator element applies the postsynaptic model and the neuron model (plainNeuronStep: the arithmetic of the neuron
// kernels), marks spikes in a bitmap in LDS whose words are the step's recording words, and appends them to the
// population's queue in ascending neuron index through the look-back the neuron kernels use.  The other populations run the
// code of the several-neurons-per-lane neuron kernel in work-groups of their own, which share the compute units with the
// layer's (four wavefronts each: a compute unit holds twelve of this kernel's), so their chains of dependent accesses
// overlap the layer's instead of adding to them.  The source's spike bitmap is double-buffered by step parity: the layer reads
// last step's spikes while this step's are written in the same launch.
#pragma once

namespace
{
struct ConvStepEpilogue
{
    PlainNeuron constants;                      // of the layer's target population, read once
    uint32_t psmKind, numCS; float psmInit, psmDecay;
    GLOBAL_AS float *var0, *var1, *outPost;     // of this batch
    uint32_t *spikeBits;                        // LDS: bit i = neuron (first neuron of the block + i) fired
    uint32_t ow, oc;
    float dt, inject;
    float l0[16], l1[16], lin[16];

    // a lane's 16 elements of a tile are pixels x0 + 8 (v / 4) + 4 half + v % 4 of output row y, channel o
    __device__ __forceinline__ void prefetch(uint32_t, uint32_t y, uint32_t x0, uint32_t o, uint32_t half)
    {
        #pragma unroll
        for(int v = 0; v < 16; v++) {
            const uint32_t x = x0 + 8 * (v / 4) + 4 * half + (v % 4);
            const bool valid = (x < ow && o < oc);
            const size_t i = valid ? ((size_t)y * ow + x) * oc + o : 0;
            l0[v] = var0[i]; l1[v] = var1[i]; lin[v] = outPost[i];
        }
    }
    __device__ __forceinline__ void finish(const f32x16 &acc, uint32_t r, uint32_t y, uint32_t x0, uint32_t o, uint32_t half)
    {
        const uint32_t lane = threadIdx.x & (WAVE - 1), col = lane & 31;
        #pragma unroll
        for(int v = 0; v < 16; v++) {
            const uint32_t x = x0 + 8 * (v / 4) + 4 * half + (v % 4);
            const bool valid = (x < ow && o < oc);
            bool spiked = false;
            if(valid) {
                const size_t i = ((size_t)y * ow + x) * oc + o;
                // postsynaptic model on this step's input: the presynaptic update's additions to outPost, as one sum
                // (neuronUpdateGroupMerged.cc:66-137; ExpCurr postsynapticModels.h:91-106, DeltaCurr :118-126)
                float linSyn = lin[v] + acc[v];
                float Isyn = 0;
                if(psmKind == GENNMI_PSM_EXPCURR) {
                    Isyn += psmInit * linSyn;
                    linSyn *= psmDecay;
                }
                else {
                    Isyn += linSyn;
                    linSyn = 0.0f;
                }
                outPost[i] = linSyn;
                if(numCS) { Isyn += inject; }
                float v0 = l0[v], v1 = l1[v];
                spiked = plainNeuronStep(constants, Isyn, dt, v0, v1);
                var0[i] = v0; var1[i] = v1;
            }
            // the 32 lanes of a half hold 32 consecutive neurons: their ballot goes into the block's bitmap
            const unsigned long long ballot = __ballot(spiked);
            if(col == 0) {
                const uint32_t bits = (uint32_t)(ballot >> (lane & 32));
                if(bits) {
                    const uint32_t base = (r * ow + x) * oc + (o - col);        // relative to the block's first neuron
                    const uint32_t word = base >> 5, shift = base & 31;
                    atomicOr(&spikeBits[word], bits << shift);
                    if(shift && (bits >> (32 - shift))) { atomicOr(&spikeBits[word + 1], bits >> (32 - shift)); }
                }
            }
        }
    }
};

constexpr int CONV_STEP_THREADS = BLOCK;

__global__ __launch_bounds__(CONV_STEP_THREADS, 3)
void convStepKernel(const ConvMfmaDev * __restrict__ conv, const NeuronGroupDev * __restrict__ target, const NeuronGroupDev * __restrict__ rest,
                    uint32_t numBatches, StepArgs args, float dt, unsigned long long *agg, unsigned long long *restAgg, uint32_t *errorFlag,
                    unsigned long long *eventCounter)
{
    extern __shared__ float shConvM[];
    __shared__ uint32_t shWaveTotal[CONV_STEP_THREADS / WAVE];
    __shared__ uint32_t shPrefix;
    __shared__ unsigned long long shWaveEvents[CONV_STEP_THREADS / WAVE];
    const Resolved st = resolve(args, dt);
    const ConvMfmaDev &G = conv[0];
    const uint32_t ow = (uint32_t)G.g.conv[6], oc = (uint32_t)G.g.conv[7], oh = (uint32_t)G.g.conv[5];
    const uint32_t convBlocks = (oh + G.rowsPerBlock - 1) / G.rowsPerBlock;
    if(blockIdx.x >= convBlocks * numBatches) {
        // ---- every other population: the code of the several-neurons-per-lane neuron kernel
        const uint32_t id = blockIdx.x - convBlocks * numBatches;
        const uint32_t batch = id / G.restBlocks, b = id - batch * G.restBlocks;
        if(G.restNeuronsPerLane == 8) { neuronBulkBody<8, CONV_STEP_THREADS>(rest[b], b, G.restBlocks, st, dt, restAgg, errorFlag, batch, numBatches); }
        else if(G.restNeuronsPerLane == 4) { neuronBulkBody<4, CONV_STEP_THREADS>(rest[b], b, G.restBlocks, st, dt, restAgg, errorFlag, batch, numBatches); }
        else if(G.restNeuronsPerLane == 2) { neuronBulkBody<2, CONV_STEP_THREADS>(rest[b], b, G.restBlocks, st, dt, restAgg, errorFlag, batch, numBatches); }
        else { neuronBulkBody<1, CONV_STEP_THREADS>(rest[b], b, G.restBlocks, st, dt, restAgg, errorFlag, batch, numBatches); }
        return;
    }
    // ---- the layer (consecutive work-groups, which go to consecutive XCDs, differ in batch)
    const uint32_t batch = blockIdx.x % numBatches, rowGroup = blockIdx.x / numBatches;
    const gennmi_neuron_update_group_t &t = target[0].g;
    const uint32_t n = t.numNeurons;
    const uint32_t firstNeuron = rowGroup * G.rowsPerBlock * ow * oc;
    const uint32_t blockNeurons = min(G.rowsPerBlock, oh - rowGroup * G.rowsPerBlock) * ow * oc;
    const uint32_t words = (blockNeurons + 31) / 32;
    uint32_t *spikeBits = reinterpret_cast<uint32_t*>(shConvM + convMfmaLdsFloats(G));
    for(uint32_t w = threadIdx.x; w < G.spikeWords; w += CONV_STEP_THREADS) { spikeBits[w] = 0u; }     // (a barrier follows inside convMfmaBlock)

    ConvStepEpilogue epilogue{plainNeuronOf(t), t.psm[0].kind, t.numCS, t.psm[0].init, t.psm[0].expDecay, asGlobal(t.var0) + (size_t)batch * n,
                              asGlobal(t.var1) + (size_t)batch * n, asGlobal(t.psm[0].outPost) + (size_t)batch * n,
                              spikeBits, ow, oc, dt, t.numCS ? t.cs[0].amp : 0.0f, {}, {}, {}};
    convMfmaBlock<CONV_STEP_THREADS>(G, rowGroup, batch, st.epoch, shConvM, epilogue, eventCounter, shWaveEvents);
    __syncthreads();

    // ---- the block's spikes, in ascending neuron index: thread k owns the words [k * per, (k + 1) * per) of the bitmap
    const uint32_t lane = threadIdx.x & (WAVE - 1), wave = threadIdx.x / WAVE;
    const uint32_t per = (words + CONV_STEP_THREADS - 1) / CONV_STEP_THREADS;
    const uint32_t wBegin = min(threadIdx.x * per, words), wEnd = min(wBegin + per, words);
    uint32_t mine = 0;
    for(uint32_t w = wBegin; w < wEnd; w++) {
        const uint32_t bits = spikeBits[w];
        mine += __popc(bits);
        // the bitmap's words are the recording words of the step (every word of the step is written: nothing to clear)
        if(t.recordSpk) { t.recordSpk[((size_t)st.recT * numBatches + batch) * ((n + 31) / 32) + (firstNeuron >> 5) + w] = bits; }
    }
    uint32_t scan = mine;       // inclusive scan over the wave, then over the waves
    for(int off = 1; off < WAVE; off <<= 1) { const uint32_t up = __shfl_up(scan, off, WAVE); if(lane >= (uint32_t)off) { scan += up; } }
    if(lane == WAVE - 1) { shWaveTotal[wave] = scan; }
    __syncthreads();
    uint32_t blockCount = 0, waveOffset = 0;
    #pragma unroll
    for(uint32_t w = 0; w < CONV_STEP_THREADS / WAVE; w++) {
        const uint32_t c = shWaveTotal[w];
        if(w < wave) { waveOffset += c; }
        blockCount += c;
    }
    unsigned long long *groupAgg = agg + (size_t)convBlocks * numBatches;
    const uint32_t prefix = blockQueueOffset(blockCount, rowGroup, convBlocks, (size_t)batch * convBlocks, agg, groupAgg, (uint32_t)(st.epoch + 1), &shPrefix, errorFlag);
    if(prefix == 0xFFFFFFFFu) { return; }
    uint32_t position = prefix + waveOffset + scan - mine;
    GLOBAL_AS uint32_t *queue = asGlobal(t.spk) + (size_t)batch * n;
    for(uint32_t w = wBegin; w < wEnd; w++) {
        uint32_t bits = spikeBits[w];
        while(bits) {
            const uint32_t bit = __ffs(bits) - 1;
            bits &= bits - 1;
            queue[position++] = firstNeuron + w * 32 + bit;
        }
    }
    if(rowGroup == convBlocks - 1 && threadIdx.x == 0) { t.spkCnt[batch] = prefix + blockCount; }
    // the work-group's synaptic events, one atomic, behind which nothing waits (shWaveEvents was written before the barrier
    // that followed the products)
    if(threadIdx.x == 0) {
        unsigned long long events = 0;
        #pragma unroll
        for(uint32_t w = 0; w < CONV_STEP_THREADS / WAVE; w++) { events += shWaveEvents[w]; }
        if(events) { addEvents(eventCounter, events); }
    }
}
}   // namespace