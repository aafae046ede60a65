/*
 * genn_mi355x_kernel_support.h — device-side building blocks of the kernels the MI355X backend GENERATES for model code
 * the device library does not implement itself (arbitrary neuron / postsynaptic / weight-update snippets).
 *
 * The generated translation unit holds the model's code, printed by GeNN's own environments into the skeletons the
 * backend emits; what is not model-specific lives here so that it is written (and reviewed) once:
 *   - the block table that maps a work-group to (group of a merged group, first element, place among the group's blocks)
 *     — the reference bisects a table of start IDs per merged group instead (backendSIMT.h:244-323);
 *   - ordered spike compaction: wave ballot -> in-wave rank, LDS -> in-block rank, tagged look-back over per-block counts
 *     -> position in the population's queue.  Queues come out in ascending neuron index, the order of the reference's
 *     SingleThreadedCPU backend (single_threaded_cpu/backend.cc:321, 2119-2133); its SIMT backends append with a
 *     shared-memory atomicAdd in arbitrary order (backendSIMT.cc:1931-1956);
 *   - the fp32 scatter-add of addToPost / addToPostDelay / addToPre (backendSIMT.cc getAtomic).
 * gfx950 only: 64-wide wavefronts, work-groups of 256 threads.
 */
#ifndef GENN_MI355X_KERNEL_SUPPORT_H
#define GENN_MI355X_KERNEL_SUPPORT_H

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace gennmi_kernel
{
constexpr int BLOCK = 256;
constexpr int WAVE = 64;
constexpr uint32_t SPIN_LIMIT = 1u << 22;       // polls a work-group waits for another one before it gives up

struct BlockEntry
{
    uint32_t group;             // index of the group within its merged group
    uint32_t firstId;           // first element this work-group handles (neuron kernels) or 0
    uint32_t blockInGroup;      // place of this work-group among the group's work-groups
    uint32_t blocksInGroup;
};

struct QueueSlot
{
    uint32_t position;          // where this lane's neuron goes in the queue (valid if it fired)
    uint32_t total;             // entries of the whole population (valid in the population's last work-group)
    bool writeTotal;            // this thread stores the count
    bool ok;                    // false: a bounded wait expired, the error flag is raised, nothing may be written
    unsigned long long ballot;  // which lanes of this wavefront fired
};

// Position of every firing lane in its population's queue.  All threads of the work-group call this, once per launch
// and population; `counts` / `groupTotals` hold one 64-bit word per work-group of the launch, tagged with `tag` (a value
// that differs from launch to launch and is never 0), so nothing is ever cleared.
__device__ inline QueueSlot orderedSlot(bool flag, uint32_t localBlock, uint32_t numBlocks, size_t aggBase,
                                        unsigned long long *counts, unsigned long long *groupTotals, uint32_t tag, uint32_t *errorFlag)
{
    __shared__ uint32_t shCount[BLOCK / WAVE];
    __shared__ uint32_t shOffset;
    const uint32_t lane = threadIdx.x & (WAVE - 1);
    const uint32_t wave = threadIdx.x / WAVE;
    QueueSlot slot;
    slot.ballot = __ballot(flag);
    const uint32_t laneRank = __popcll(slot.ballot & ((1ull << lane) - 1ull));
    if(lane == 0) { shCount[wave] = __popcll(slot.ballot); }
    __syncthreads();
    uint32_t blockCount = 0, waveOffset = 0;
    #pragma unroll
    for(uint32_t w = 0; w < BLOCK / WAVE; w++) {
        const uint32_t c = shCount[w];
        if(w < wave) { waveOffset += c; }
        blockCount += c;
    }
    if(threadIdx.x == 0) {
        __hip_atomic_store(&counts[aggBase + localBlock], ((unsigned long long)tag << 32) | blockCount, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    const bool last = (localBlock == numBlocks - 1);
    if(wave == 0) {
        // work-groups of a population form groups of 64: a work-group's offset is the sum of the counts of the earlier
        // work-groups of its group plus the published totals of the earlier groups; every wait is for a value that depends
        // only on other work-groups having published their own count
        const uint32_t group = localBlock / WAVE, inGroup = localBlock % WAVE;
        const size_t groupBase = aggBase + (size_t)group * WAVE;
        bool ok = true;
        auto waitFor = [&](const unsigned long long *p) -> uint32_t {
            uint32_t spins = 0;
            while(true) {
                const unsigned long long a = __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                if((uint32_t)(a >> 32) == tag) { return (uint32_t)a; }
                if(++spins > SPIN_LIMIT) { ok = false; return 0u; }
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
            shOffset = sum;
        }
    }
    __syncthreads();
    const uint32_t prefix = shOffset;
    slot.ok = (prefix != 0xFFFFFFFFu);
    slot.position = prefix + waveOffset + laneRank;
    slot.total = prefix + blockCount;
    slot.writeTotal = last && threadIdx.x == 0;
    __syncthreads();            // the shared words are reused by the next call
    return slot;
}

// the ballot is the recording bitfield of the step (bit i % 32 of word i / 32, runtime.cc:855-913): every word of the step is
// overwritten, so there is nothing to clear and no atomicOr (cf. backendSIMT.cc:1948-1953)
__device__ inline void recordBallot(uint32_t *recordWords, uint32_t id, bool inRange, unsigned long long ballot)
{
    const uint32_t lane = threadIdx.x & (WAVE - 1);
    if((lane & 31) == 0 && inRange) { recordWords[id >> 5] = (uint32_t)(ballot >> (lane & 32)); }
}

__device__ inline void addScalar(float *address, float value) { unsafeAtomicAdd(address, value); }
__device__ inline void addScalar(double *address, double value) { unsafeAtomicAdd(address, value); }
}   // namespace gennmi_kernel

#endif
