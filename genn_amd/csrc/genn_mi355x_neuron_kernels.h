// Part of libgenn_mi355x.so: included by genn_mi355x.hip only (one translation unit).
#ifndef GENN_MI355X_NEURON_KERNELS_H
#define GENN_MI355X_NEURON_KERNELS_H

namespace
{
// PoissonExp current source (currentSourceModels.h:100-129): the snippet's loop draws uniforms until their product falls to
// ExpMinusLambda; here the draws of (neuron, step) are the words of counter-based generator calls, so the result does not
// depend on the launch geometry or on which plan steps the network.
__device__ __forceinline__ uint32_t poissonExpCount(const gennmi_cs_t &cs, size_t bi, unsigned long long epoch)
{
    const gennmi_rows::Stream s{(uint32_t)cs.seed, (uint32_t)(cs.seed >> 32), cs.stream};
    float p = 1.0f;
    uint32_t numSpikes = 0;
    for(uint32_t call = 0; ; call++) {
        const gennmi_rows::Words r = gennmi_rows::philox4x32((uint32_t)bi, (uint32_t)epoch, call, s.stream, s.k0, s.k1);
        bool done = false;
        #pragma unroll
        for(int w = 0; w < 4 && !done; w++) {
            numSpikes++;
            p *= gennmi_rows::uniformHalfOpen(r.w[w]);
            done = !(p > cs.expMinusLambda);
        }
        if(done) { break; }
    }
    return numSpikes - 1;
}

// one step of the source whose state the caller holds: returns the injected value, leaves the decayed one in `current`
__device__ __forceinline__ float poissonExpStep(const gennmi_cs_t &cs, float &current, size_t bi, unsigned long long epoch)
{
    const float value = current + cs.init * (float)poissonExpCount(cs, bi, epoch);
    current = value * cs.expDecay;
    return value;
}

__device__ __forceinline__ float poissonExpInject(const gennmi_cs_t &cs, GLOBAL_AS float *current, size_t bi, unsigned long long epoch)
{
    float state = current[bi];
    const float value = poissonExpStep(cs, state, bi, epoch);
    current[bi] = state;
    return value;
}

// ------------------------------------------------------------------------------------------------
// Offset of a block's entries in its population's queue: the block publishes its count, then (wave 0) sums the counts of
// the earlier blocks of its group of 64 and the published totals of the earlier groups.  Every thread of the block calls
// this between two barriers of its own; returns 0xFFFFFFFF after a bounded wait expired (error flag raised).
// (`published`: the caller has stored the block's count itself, earlier — see publishBlockCount)
__device__ __forceinline__ void publishBlockCount(uint32_t blockCount, uint32_t localBlock, size_t aggBase, unsigned long long *counts, uint32_t tag)
{
    if(threadIdx.x == 0) {
        __hip_atomic_store(&counts[aggBase + localBlock], ((unsigned long long)tag << 32) | blockCount, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
}
__device__ __forceinline__ uint32_t blockQueueOffset(uint32_t blockCount, uint32_t localBlock, uint32_t numBlocks, size_t aggBase,
                                                    unsigned long long *counts, unsigned long long *groupTotals, uint32_t tag,
                                                    uint32_t *shOffset, uint32_t *errorFlag, bool published = false)
{
    const uint32_t lane = threadIdx.x & (WAVE - 1);
    const uint32_t wave = threadIdx.x / WAVE;
    if(threadIdx.x == 0 && !published) {
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
            if(!allOk) { raiseErrorFlag(errorFlag); sum = 0xFFFFFFFFu; }
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
    // what the update leaves to be stored (see storeState below)
    float l0 = 0, l1 = 0, preTrace = 0, postTrace = 0;
    float lin[GENNMI_MAX_PSM];
    #pragma unroll
    for(uint32_t m = 0; m < GENNMI_MAX_PSM; m++) { lin[m] = 0.0f; }
    if(i < n) {
        // order of operations: neuronUpdateGroupMerged.cc:552-773 — PSMs, current sources, sim code,
        // WU pre/post dynamics, threshold, then (on a spike) WU pre/post spike code, sT, reset
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
            float front[GENNMI_MAX_PSM], inj[GENNMI_MAX_CS], rev[GENNMI_MAX_PRE_OUTPUT];
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
                           : (g.cs[c].kind == GENNMI_CS_ARRAY) ? asGlobal(g.cs[c].array)[(size_t)modStep(st.epoch, g.cs[c].arraySteps) * n + i]
                                                               : poissonExpInject(g.cs[c], asGlobal(g.cs[c].current), bi, st.epoch);
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
        if(g.preTrace) { preTrace = g.preTrace[bi] * g.preDecay; }
        if(g.postTrace) { postTrace = g.postTrace[bi] * g.postDecay; }
        if(g.model == GENNMI_NEURON_LIF) { spiked = (l1 <= 0.0f && l0 >= g.params[4]); }
        else if(g.model == GENNMI_NEURON_IZHIKEVICH) { spiked = (l0 >= 29.99f); }
        else { spiked = (t >= nextTime); }       // startSpike != endSpike && t >= spikeTimes[startSpike] (neuronModels.h:274-286)
        vEvent = l0;           // spike-like event conditions see the updated V before any reset (neuronUpdateGroupMerged.cc:677-683)
        if(spiked) {
            preTrace += 1.0f; postTrace += 1.0f;
            if(g.model == GENNMI_NEURON_LIF) { l0 = g.params[5]; l1 = g.params[6]; }
        }
    }
    // The stores of the update, issued once the block's spike count is on its way (the work-groups behind this one wait for
    // that count; a wavefront queued behind the chip's store traffic before it can vote would keep them waiting).
    auto storeState = [&]() {
        if(i < n) {
            if(g.model == GENNMI_NEURON_SPIKE_SOURCE_ARRAY) {
                if(spiked) {
                    const uint32_t startSpike = g.startSpike[bi] + 1;
                    g.startSpike[bi] = startSpike;
                    G.nextSpikeTime[bi] = (startSpike != g.endSpike[bi]) ? g.spikeTimes[startSpike] : INFINITY;
                }
            }
            else {
                const uint32_t numPSM = g.numPSM, numRev = g.numPreOutput;
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
                g.var0[bi] = l0; g.var1[bi] = l1;
            }
            if(spiked && g.sT) { g.sT[bi] = t; }
            if(g.preTrace) { g.preTrace[bi] = preTrace; }
            if(g.postTrace) { g.postTrace[bi] = postTrace; }
        }
        // keep the user-visible ring pointers current (nothing in the kernels reads them)
        if(localBlock == 0 && batch == 0 && threadIdx.x < g.numPSM) {
            const gennmi_psm_t &psm = g.psm[threadIdx.x];
            if(psm.maxDenDelay && psm.denDelayPtr) { *psm.denDelayPtr = modStep(st.epoch + 1, psm.maxDenDelay); }
        }
    };

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
    if(G.spikeBitmap && (lane & 31) == 0 && i < n) { G.spikeBitmap[((st.epoch + 1) & 1) * G.bitmapStride + (size_t)batch * ((n + 31) / 32) + (i >> 5)] = (uint32_t)(ballot >> (lane & 32)); }
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
    storeState();
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
            if(!allOk) { raiseErrorFlag(errorFlag); sum = 0xFFFFFFFFu; }
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

// What the update of a plain neuron needs of its group, read once into registers: the descriptor lives in global memory, and
// behind every store the compiler would read its fields again (a store may alias anything), ten dependent scalar loads per neuron.
struct PlainNeuron
{
    uint32_t model;
    float p[7];
};
__device__ __forceinline__ PlainNeuron plainNeuronOf(const gennmi_neuron_update_group_t &g)
{
    PlainNeuron c;
    c.model = g.model;
    #pragma unroll
    for(int k = 0; k < 7; k++) { c.p[k] = g.params[k]; }
    return c;
}
// sim code, threshold and reset of a LIF (neuronModels.h:220-257) or Izhikevich (:163-186) neuron from its summed input:
// operations and their order as in neuronBody
__device__ __forceinline__ bool plainNeuronStep(const PlainNeuron &c, float Isyn, float dt, float &v0, float &v1)
{
    bool spiked;
    if(c.model == GENNMI_NEURON_LIF) {
        if(v1 <= 0.0f) {
            const float alpha = ((Isyn + c.p[0]) * c.p[1]) + c.p[2];
            v0 = alpha - (c.p[3] * (alpha - v0));
        }
        else {
            v1 -= dt;
        }
        spiked = (v1 <= 0.0f && v0 >= c.p[4]);
        if(spiked) { v0 = c.p[5]; v1 = c.p[6]; }
    }
    else {
        if(v0 >= 30.0f) {
            v0 = c.p[2];
            v1 += c.p[3];
        }
        v0 += 0.5f * (0.04f * v0 * v0 + 5.0f * v0 + 140.0f - v1 + Isyn) * dt;
        v0 += 0.5f * (0.04f * v0 * v0 + 5.0f * v0 + 140.0f - v1 + Isyn) * dt;
        v1 += c.p[0] * (c.p[1] * v0 - v1) * dt;
        if(v0 > 30.0f) { v0 = 30.0f; }
        spiked = (v0 >= 29.99f);
    }
    return spiked;
}

// (THREADS: threads of the calling work-group, all of which call; batch / numBatches: the grid's second dimension in the neuron kernels)
template<int NPL, int THREADS = BLOCK>
__device__ __forceinline__ void neuronBulkBody(const NeuronGroupDev &G, uint32_t blockInKernel, uint32_t totalNeuronBlocks,
                                               const Resolved &st, float dt, unsigned long long *agg, uint32_t *errorFlag,
                                               uint32_t batch, uint32_t numBatches)
{
    __shared__ uint32_t shWaveCount[THREADS / WAVE];
    __shared__ uint32_t shPrefix;
    const gennmi_neuron_update_group_t &g = G.g;
    const uint32_t localBlock = blockInKernel - G.startBlock;
    const uint32_t n = g.numNeurons;
    const uint32_t lane = threadIdx.x & (WAVE - 1);
    const uint32_t wave = threadIdx.x / WAVE;
    const float t = st.t;
    const uint32_t first = (localBlock * (THREADS / WAVE) + wave) * (WAVE * NPL) + lane;      // this lane's neuron in chunk 0
    const uint32_t numPSM = g.numPSM, numCS = g.numCS;
    // the group's constants and array addresses, read once (see PlainNeuron)
    const PlainNeuron constants = plainNeuronOf(g);
    const bool source = (constants.model == GENNMI_NEURON_SPIKE_SOURCE_ARRAY);
    GLOBAL_AS float *var0 = asGlobal(g.var0), *var1 = asGlobal(g.var1);
    GLOBAL_AS float *psmOut[BULK_MAX_PSM], *psmRing[BULK_MAX_PSM];
    uint32_t psmD[BULK_MAX_PSM], psmKind[BULK_MAX_PSM];
    float psmInit[BULK_MAX_PSM], psmDecay[BULK_MAX_PSM];
    #pragma unroll
    for(uint32_t m = 0; m < BULK_MAX_PSM; m++) {
        const bool have = (m < numPSM);
        psmOut[m] = have ? asGlobal(g.psm[m].outPost) : nullptr; psmRing[m] = have ? asGlobal(g.psm[m].denDelay) : nullptr;
        psmD[m] = have ? g.psm[m].maxDenDelay : 0u; psmKind[m] = have ? g.psm[m].kind : 0u;
        psmInit[m] = have ? g.psm[m].init : 0.0f; psmDecay[m] = have ? g.psm[m].expDecay : 0.0f;
    }
    const uint32_t csKind = numCS ? g.cs[0].kind : 0u, csSteps = numCS ? g.cs[0].arraySteps : 1u;
    const float csAmp = numCS ? g.cs[0].amp : 0.0f;
    GLOBAL_AS const float *csArray = numCS ? asGlobal(g.cs[0].array) : nullptr;
    uint32_t *recordSpk = g.recordSpk, *spikeBitmap = G.spikeBitmap;
    uint32_t *startSpikeArr = g.startSpike; const uint32_t *endSpikeArr = g.endSpike; const float *spikeTimesArr = g.spikeTimes;
    float *nextSpikeTime = G.nextSpikeTime;
    const size_t bitmapStride = G.bitmapStride;
    uint32_t *spkQueue = g.spk, *spkCount = g.spkCnt;
    const uint32_t groupBlocks = G.numBlocks, groupStart = G.startBlock;

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
            if(source) {
                l0[j] = asGlobal(nextSpikeTime)[bi];
            }
            else {
                l0[j] = var0[bi]; l1[j] = var1[bi];
                #pragma unroll
                for(uint32_t m = 0; m < BULK_MAX_PSM; m++) {
                    if(m < numPSM) {
                        lin[j][m] = psmOut[m][bi];
                        const uint32_t D = psmD[m];
                        if(D) { front[j][m] = psmRing[m][((size_t)batch * D + modStep(st.epoch + 1, D)) * n + i]; }
                    }
                }
                if(numCS) {
                    inj[j] = (csKind == GENNMI_CS_DC) ? csAmp : csArray[(size_t)modStep(st.epoch, csSteps) * n + i];
                }
            }
        }
    }
    // ---- update, chunk by chunk (operations and their order as in neuronBody); results stay in registers until the block's
    // spike count is on its way: work-groups behind this one wait for that count, and a wavefront that has to queue
    // behind the store traffic of the whole chip before it can vote would keep them waiting
    float outLin[NPL][BULK_MAX_PSM];
    uint32_t newStart[NPL];
    #pragma unroll
    for(int j = 0; j < NPL; j++) {
        const uint32_t i = first + j * WAVE;
        const size_t bi = (size_t)batch * n + i;
        newStart[j] = 0;
        #pragma unroll
        for(uint32_t m = 0; m < BULK_MAX_PSM; m++) { outLin[j][m] = 0.0f; }
        if(i >= n) { continue; }
        if(source) {
            spiked[j] = (t >= l0[j]);
            if(spiked[j]) { newStart[j] = startSpikeArr[bi] + 1; }
            continue;
        }
        float Isyn = 0;
        #pragma unroll
        for(uint32_t m = 0; m < BULK_MAX_PSM; m++) {
            if(m < numPSM) {
                float linSyn = lin[j][m];
                const uint32_t D = psmD[m];
                if(D) { linSyn += front[j][m]; }
                if(psmKind[m] == GENNMI_PSM_EXPCURR) {
                    Isyn += psmInit[m] * linSyn;
                    linSyn *= psmDecay[m];
                }
                else {
                    Isyn += linSyn;
                    linSyn = 0.0f;
                }
                outLin[j][m] = linSyn;
            }
        }
        if(numCS) { Isyn += inj[j]; }
        spiked[j] = plainNeuronStep(constants, Isyn, dt, l0[j], l1[j]);
    }

    // ---- ordered compaction: rank = spikes of the wave's earlier chunks + spikes of lower lanes in this chunk
    uint32_t rank[NPL];
    unsigned long long ballots[NPL];
    uint32_t waveCount = 0;
    #pragma unroll
    for(int j = 0; j < NPL; j++) {
        ballots[j] = __ballot(spiked[j]);
        rank[j] = waveCount + __popcll(ballots[j] & ((1ull << lane) - 1ull));
        waveCount += __popcll(ballots[j]);
    }
    if(lane == 0) { shWaveCount[wave] = waveCount; }
    __syncthreads();
    uint32_t blockCount = 0, waveOffset = 0;
    #pragma unroll
    for(uint32_t w = 0; w < THREADS / WAVE; w++) {
        const uint32_t c = shWaveCount[w];
        if(w < wave) { waveOffset += c; }
        blockCount += c;
    }
    unsigned long long *groupAgg = agg + (size_t)totalNeuronBlocks * numBatches;
    const size_t aggBase = (size_t)batch * totalNeuronBlocks + groupStart;
    publishBlockCount(blockCount, localBlock, aggBase, agg, (uint32_t)(st.epoch + 1));

    // ---- state, recording words and bitmap
    #pragma unroll
    for(int j = 0; j < NPL; j++) {
        const uint32_t i = first + j * WAVE;
        const size_t bi = (size_t)batch * n + i;
        if(i >= n) { continue; }
        if(recordSpk && (lane & 31) == 0) {
            const uint32_t words = (n + 31) / 32;
            recordSpk[((size_t)st.recT * numBatches + batch) * words + (i >> 5)] = (uint32_t)(ballots[j] >> (lane & 32));
        }
        if(spikeBitmap && (lane & 31) == 0) { spikeBitmap[((st.epoch + 1) & 1) * bitmapStride + (size_t)batch * ((n + 31) / 32) + (i >> 5)] = (uint32_t)(ballots[j] >> (lane & 32)); }
        if(source) {
            if(spiked[j]) {
                startSpikeArr[bi] = newStart[j];
                nextSpikeTime[bi] = (newStart[j] != endSpikeArr[bi]) ? spikeTimesArr[newStart[j]] : INFINITY;
            }
            continue;
        }
        #pragma unroll
        for(uint32_t m = 0; m < BULK_MAX_PSM; m++) {
            if(m < numPSM) {
                const uint32_t D = psmD[m];
                if(D) { psmRing[m][((size_t)batch * D + modStep(st.epoch + 1, D)) * n + i] = 0.0f; }
                // (an input that is the same bits as it was read — a DeltaCurr input that received nothing: zero in, zero out —
                // is not written again: in a quiet step that is most of a population's 4 bytes per neuron)
                if(__float_as_uint(outLin[j][m]) != __float_as_uint(lin[j][m])) { psmOut[m][bi] = outLin[j][m]; }
            }
        }
        var0[bi] = l0[j]; var1[bi] = l1[j];
    }
    if(localBlock == 0 && batch == 0 && threadIdx.x < g.numPSM) {
        const gennmi_psm_t &psm = g.psm[threadIdx.x];
        if(psm.maxDenDelay && psm.denDelayPtr) { *psm.denDelayPtr = modStep(st.epoch + 1, psm.maxDenDelay); }
    }

    const uint32_t prefix = blockQueueOffset(blockCount, localBlock, groupBlocks, aggBase, agg, groupAgg,
                                             (uint32_t)(st.epoch + 1), &shPrefix, errorFlag, true);
    if(prefix == 0xFFFFFFFFu) { return; }
    #pragma unroll
    for(int j = 0; j < NPL; j++) {
        if(spiked[j]) { spkQueue[(size_t)batch * n + prefix + waveOffset + rank[j]] = first + j * WAVE; }
    }
    if(localBlock == groupBlocks - 1 && threadIdx.x == 0) { spkCount[batch] = prefix + blockCount; }
}

template<int NPL>
__global__ __launch_bounds__(BLOCK)
void neuronBulkKernel(const NeuronGroupDev * __restrict__ blocks, StepArgs args, float dt, unsigned long long *agg, uint32_t *errorFlag)
{
    neuronBulkBody<NPL>(blocks[blockIdx.x], blockIdx.x, gridDim.x, resolve(args, dt), dt, agg, errorFlag, blockIdx.y, gridDim.y);
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
    else { presynapticBody(preBlocks[blockIdx.x - numNeuronBlocks], blockIdx.x - numNeuronBlocks, blockIdx.y, gridDim.y, st, dt, eventCounter); }
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
// early deliveries of zero-delay synapses that have to be added or taken back after the connectivity was rewritten
struct ZeroDelayCorrection { float *target; const float *weight; float sign; uint32_t pad_; };
__global__ void zeroDelayCorrectionKernel(const ZeroDelayCorrection *fix, uint32_t count)
{
    const uint32_t k = blockIdx.x * blockDim.x + threadIdx.x;
    if(k < count) { atomicAddF32(asGlobal(fix[k].target), fix[k].sign * fix[k].weight[0]); }
}

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

}   // namespace

#endif
