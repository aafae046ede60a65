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
 *   - the fp32 scatter-add of addToPost / addToPostDelay / addToPre (backendSIMT.cc getAtomic);
 *   - for custom updates: the group of a work-group by bisection, and work-group-wide sum / maximum.
 * gfx950 only: 64-wide wavefronts, work-groups of 256 threads.
 */
#ifndef GENN_MI355X_KERNEL_SUPPORT_H
#define GENN_MI355X_KERNEL_SUPPORT_H

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "genn_mi355x.h"        // gennmi_launch_header_t: the first argument of every generated kernel

namespace gennmi_kernel
{
constexpr int BLOCK = 256;
constexpr int WAVE = 64;

// the values of the step a launch belongs to: by value in the header (a launch made when it was asked for) or in a device
// table (a launch replayed from a captured graph, whose arguments are the same at every replay)
__device__ inline gennmi_step_entry_t stepEntry(const gennmi_launch_header_t &header)
{
    return header.steps ? header.steps[header.k] : header.inlineEntry;
}

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
// that differs from launch to launch and is never 0), so nothing is ever cleared.  A work-group polls another one's word at
// most `spinLimit` times; then it raises the error flag and leaves (slot.ok == false) instead of hanging.
__device__ inline QueueSlot orderedSlot(bool flag, uint32_t localBlock, uint32_t numBlocks, size_t aggBase,
                                        unsigned long long *counts, unsigned long long *groupTotals, uint32_t tag, uint32_t *errorFlag,
                                        uint32_t spinLimit)
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
                if(++spins > spinLimit) { ok = false; return 0u; }
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

// ---- random numbers of simulation code (gennrand_* in neuron, current-source and postsynaptic snippets).
// The reference keeps a generator state per neuron in memory (XORWOW on its SIMT backends, one host mt19937 on the CPU
// backend: no two of its backends draw the same numbers, so there is nothing bit-exact to match).  Here a draw is a word of
// Philox4x32-10 (Salmon, Moraes, Dror, Shaw, SC'11) under key = the model's seed with counter = (batch * neurons + neuron,
// timestep, number of the call within the step, one stream per population): no state in memory, the same numbers whatever
// the launch geometry.
struct Rng
{
    uint32_t k0, k1, element, stepLow, stepHighAndCall, stream;
    uint32_t w0, w1, w2, w3, left;
};

__device__ inline void philox4x32(uint32_t c0, uint32_t c1, uint32_t c2, uint32_t c3, uint32_t k0, uint32_t k1, uint32_t &o0, uint32_t &o1, uint32_t &o2, uint32_t &o3)
{
    #pragma unroll
    for(int round = 0; round < 10; round++) {
        const uint32_t hi0 = __umulhi(0xD2511F53u, c0), lo0 = 0xD2511F53u * c0;
        const uint32_t hi1 = __umulhi(0xCD9E8D57u, c2), lo1 = 0xCD9E8D57u * c2;
        c0 = hi1 ^ c1 ^ k0;
        c1 = lo1;
        c2 = hi0 ^ c3 ^ k1;
        c3 = lo0;
        k0 += 0x9E3779B9u;
        k1 += 0xBB67AE85u;
    }
    o0 = c0; o1 = c1; o2 = c2; o3 = c3;
}

// (element: a neuron of a batch, or a synapse of a batch — up to 2^44 of them; its high bits travel above the stream number)
__device__ inline Rng rngBegin(unsigned long long seed, uint32_t stream, unsigned long long element, unsigned long long step)
{
    Rng r;
    r.k0 = (uint32_t)seed; r.k1 = (uint32_t)(seed >> 32);
    r.element = (uint32_t)element; r.stepLow = (uint32_t)step; r.stepHighAndCall = (uint32_t)(step >> 32) << 16;
    r.stream = stream | ((uint32_t)(element >> 32) << 20);
    r.w0 = r.w1 = r.w2 = r.w3 = 0; r.left = 0;
    return r;
}

// next 32-bit word of the neuron's sequence for this step (four per generator call; at most 65,536 calls per neuron and step)
__device__ inline uint32_t rngWord(Rng &r)
{
    if(r.left == 0) {
        philox4x32(r.element, r.stepLow, r.stepHighAndCall, r.stream, r.k0, r.k1, r.w0, r.w1, r.w2, r.w3);
        r.stepHighAndCall = (r.stepHighAndCall & 0xFFFF0000u) | ((r.stepHighAndCall + 1u) & 0xFFFFu);
        r.left = 4;
    }
    const uint32_t word = r.w0;
    r.w0 = r.w1; r.w1 = r.w2; r.w2 = r.w3;
    r.left--;
    return word;
}

__device__ inline float rngUniform(Rng &r) { return ((float)(rngWord(r) >> 8) + 0.5f) * (1.0f / 16777216.0f); }          // (0, 1)
__device__ inline float rngExponential(Rng &r) { return -logf(rngUniform(r)); }
__device__ inline float rngNormal(Rng &r)
{
    // Box-Muller; the sine branch is not kept (a neuron that wants two normals pays two pairs of words)
    const float radius = sqrtf(-2.0f * logf(rngUniform(r)));
    return radius * cospif(2.0f * ((float)(rngWord(r) >> 8) * (1.0f / 16777216.0f)));
}
__device__ inline float rngLogNormal(Rng &r, float mean, float sd) { return expf(mean + sd * rngNormal(r)); }
// Marsaglia & Tsang (2000) for shape >= 1; shape < 1 through gamma(a + 1) * u^(1/a)
__device__ inline float rngGamma(Rng &r, float a)
{
    const float boost = (a < 1.0f) ? 1.0f : 0.0f;
    const float d = (a + boost) - (1.0f / 3.0f);
    const float c = 1.0f / sqrtf(9.0f * d);
    while(true) {
        const float x = rngNormal(r);
        float v = 1.0f + c * x;
        if(v <= 0.0f) { continue; }
        v = v * v * v;
        const float u = rngUniform(r);
        if(u < 1.0f - 0.0331f * (x * x) * (x * x) || logf(u) < 0.5f * x * x + d * (1.0f - v + logf(v))) {
            return (boost != 0.0f) ? d * v * powf(rngUniform(r), 1.0f / a) : d * v;
        }
    }
}
// Binomial(n, p) by inversion of the CDF from k = 0, in slices of n short enough that (1 - p)^slice stays a normal double
__device__ inline uint32_t rngBinomial(Rng &r, uint32_t n, float p)
{
    if(!(p > 0.0f) || n == 0) { return 0; }
    if(p >= 1.0f) { return n; }
    const bool flip = p > 0.5f;
    const double pp = flip ? 1.0 - (double)p : (double)p;
    const double logQ = log1p(-pp);
    const uint32_t maxSlice = (uint32_t)fmin(4.0e9, fmax(1.0, floor(-600.0 / logQ)));
    const double ratio = pp / (1.0 - pp);
    uint32_t total = 0, done = 0;
    while(done < n) {
        const uint32_t m = min(maxSlice, n - done);
        const uint32_t hi = rngWord(r), lo = rngWord(r);
        double u = ((double)hi * 4294967296.0 + (double)lo + 0.5) * (1.0 / 18446744073709551616.0);
        double pmf = exp((double)m * logQ);
        uint32_t k = 0;
        while(u > pmf && k < m) {
            u -= pmf;
            k++;
            pmf *= ratio * (double)(m - k + 1) / (double)k;
        }
        total += k;
        done += m;
    }
    return flip ? n - total : total;
}

__device__ inline void addScalar(float *address, float value) { unsafeAtomicAdd(address, value); }
__device__ inline void addScalar(double *address, double value) { unsafeAtomicAdd(address, value); }

// ---- custom updates ---------------------------------------------------------------------------------------------------
// Per-synapse custom updates can span millions of work-groups, so their kernels do not carry a table entry per
// work-group: `starts` holds, per group of a merged group, the first work-group of the group (count + 1 entries,
// ascending); the group of a work-group is found by bisection (backendSIMT.h:244-323 does the same over thread ids).
__device__ inline uint32_t groupOfBlock(const uint32_t *starts, uint32_t count, uint32_t block)
{
    uint32_t lo = 0, hi = count;
    while(hi - lo > 1) {
        const uint32_t mid = (lo + hi) / 2;
        if(block >= starts[mid]) { lo = mid; } else { hi = mid; }
    }
    return lo;
}

// Reductions over the neurons of a population (custom update variables with REDUCE_NEURON_* access): every thread of the
// work-group brings its partial result, every thread leaves with the work-group's.  Wave shuffles, then one LDS word per
// wave.  A sum's order differs from the CPU backend's index order, so fp32 sums agree to rounding, not bit for bit.
template<typename T, typename Op>
__device__ inline T blockReduce(T value, Op op)
{
    __shared__ T shWave[BLOCK / WAVE];
    for(int o = WAVE / 2; o > 0; o >>= 1) { value = op(value, __shfl_xor(value, o, WAVE)); }
    __syncthreads();                                    // (the words may still be read from an earlier reduction)
    if((threadIdx.x & (WAVE - 1)) == 0) { shWave[threadIdx.x / WAVE] = value; }
    __syncthreads();
    T result = shWave[0];
    for(int w = 1; w < BLOCK / WAVE; w++) { result = op(result, shWave[w]); }
    return result;
}
template<typename T> __device__ inline T blockReduceSum(T value) { return blockReduce(value, [](T a, T b) { return a + b; }); }
template<typename T> __device__ inline T blockReduceMax(T value) { return blockReduce(value, [](T a, T b) { return (a > b) ? a : b; }); }
__device__ inline float blockReduceMax(float value) { return blockReduce(value, [](float a, float b) { return fmaxf(a, b); }); }
__device__ inline double blockReduceMax(double value) { return blockReduce(value, [](double a, double b) { return fmax(a, b); }); }
}   // namespace gennmi_kernel

#endif
