// Counter-based random rows and values, shared by the initialisation kernels (which store them) and the procedural
// presynaptic kernel (which regenerates them for every spike): device code only, included by both translation units.
//
// Every draw is Philox4x32-10 of (seed, stream, row or element, draw number), so whoever asks for synapse k of row r, or for
// element e of a variable, gets the same answer whatever the launch geometry and however often it asks.
#ifndef GENN_MI355X_ROWS_H
#define GENN_MI355X_ROWS_H

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "genn_mi355x.h"

namespace gennmi_rows
{
constexpr int WAVE = 64;

// Philox4x32-10 (Salmon, Moraes, Dror, Shaw: "Parallel random numbers: as easy as 1, 2, 3", SC'11)
struct Words { uint32_t w[4]; };

__host__ __device__ inline uint32_t mulHi(uint32_t a, uint32_t b) { return (uint32_t)(((unsigned long long)a * b) >> 32); }

__host__ __device__ inline Words philox4x32(uint32_t c0, uint32_t c1, uint32_t c2, uint32_t c3, uint32_t k0, uint32_t k1)
{
    #pragma unroll
    for(int round = 0; round < 10; round++) {
        const uint32_t hi0 = mulHi(0xD2511F53u, c0), lo0 = 0xD2511F53u * c0;
        const uint32_t hi1 = mulHi(0xCD9E8D57u, c2), lo1 = 0xCD9E8D57u * c2;
        c0 = hi1 ^ c1 ^ k0;
        c1 = lo1;
        c2 = hi0 ^ c3 ^ k1;
        c3 = lo0;
        k0 += 0x9E3779B9u;
        k1 += 0xBB67AE85u;
    }
    return Words{{c0, c1, c2, c3}};
}

// A stream of draws: key = the 64-bit seed, counter = (index low, index high, sub-counter, stream number).
struct Stream
{
    uint32_t k0, k1, stream;
    __host__ __device__ Words at(unsigned long long index, uint32_t sub) const
    {
        return philox4x32((uint32_t)index, (uint32_t)(index >> 32), sub, stream, k0, k1);
    }
};

__device__ __forceinline__ float uniformHalfOpen(uint32_t x) { return (float)(x >> 8) * (1.0f / 16777216.0f); }              // [0, 1)
__device__ __forceinline__ float uniformOpen(uint32_t x) { return ((float)(x >> 8) + 0.5f) * (1.0f / 16777216.0f); }         // (0, 1)

// four standard normals from four words (Box-Muller, both branches)
__device__ __forceinline__ void normals(const Words &r, float n[4])
{
    #pragma unroll
    for(int p = 0; p < 2; p++) {
        const float radius = sqrtf(-2.0f * logf(uniformOpen(r.w[2 * p])));
        float s, c;
        sincospif(2.0f * uniformHalfOpen(r.w[2 * p + 1]), &s, &c);
        n[2 * p] = radius * c;
        n[2 * p + 1] = radius * s;
    }
}

// ---- wave64 scans
__device__ __forceinline__ uint32_t waveInclusiveScan(uint32_t v, int lane)
{
    #pragma unroll
    for(int d = 1; d < WAVE; d <<= 1) {
        const uint32_t o = __shfl_up(v, d, WAVE);
        if(lane >= d) { v += o; }
    }
    return v;
}
__device__ __forceinline__ double waveInclusiveScan(double v, int lane)
{
    #pragma unroll
    for(int d = 1; d < WAVE; d <<= 1) {
        const double o = __shfl_up(v, d, WAVE);
        if(lane >= d) { v += o; }
    }
    return v;
}

struct VarInit { uint32_t snippet; float p[4]; double p64[2]; };

// value of element `e` whose group of four shares the Philox call `r` (attempt 0); slot = e % 4
__device__ __forceinline__ float drawValue(const VarInit &v, const Stream &s, unsigned long long group, int slot, const Words &r, const float n[4])
{
    switch(v.snippet) {
    case GENNMI_INIT_CONSTANT:
        return v.p[0];
    case GENNMI_INIT_UNIFORM: {
        const float scale = v.p[1] - v.p[0];
        return v.p[0] + (uniformHalfOpen(r.w[slot]) * scale);
    }
    case GENNMI_INIT_NORMAL:
        return v.p[0] + (n[slot] * v.p[1]);
    case GENNMI_INIT_NORMAL_CLIPPED:
    case GENNMI_INIT_NORMAL_CLIPPED_DELAY: {
        float value = v.p[0] + (n[slot] * v.p[1]);
        for(uint32_t attempt = 1; value > v.p[3] || value < v.p[2]; attempt++) {
            float retry[4];
            normals(s.at(group, attempt), retry);
            value = v.p[0] + (retry[slot] * v.p[1]);
        }
        return (v.snippet == GENNMI_INIT_NORMAL_CLIPPED_DELAY) ? rintf(value) : value;
    }
    case GENNMI_INIT_EXPONENTIAL:
        return v.p[0] * -logf(uniformOpen(r.w[slot]));
    default:
        return 0.0f;
    }
}


// value of element e of a variable initialised with `v` from stream `s` (what initVarKernel stores there); the
// snippets that draw per element rather than per group of four (Gamma, Binomial) are not available here
__device__ __forceinline__ float valueAt(const VarInit &v, const Stream &s, unsigned long long e)
{
    if(v.snippet == GENNMI_INIT_CONSTANT) { return v.p[0]; }
    const unsigned long long group = e >> 2;
    const Words r = s.at(group, 0);
    float n[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    if(v.snippet == GENNMI_INIT_NORMAL || v.snippet == GENNMI_INIT_NORMAL_CLIPPED || v.snippet == GENNMI_INIT_NORMAL_CLIPPED_DELAY) { normals(r, n); }
    return drawValue(v, s, group, (int)(e & 3), r, n);
}

// elements e0..e0+3 at once (e0 a multiple of four): the four share one generator call
__device__ __forceinline__ void valuesAt4(const VarInit &v, const Stream &s, unsigned long long e0, float out[4])
{
    if(v.snippet == GENNMI_INIT_CONSTANT) { out[0] = out[1] = out[2] = out[3] = v.p[0]; return; }
    const unsigned long long group = e0 >> 2;
    const Words r = s.at(group, 0);
    float n[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    if(v.snippet == GENNMI_INIT_NORMAL || v.snippet == GENNMI_INIT_NORMAL_CLIPPED || v.snippet == GENNMI_INIT_NORMAL_CLIPPED_DELAY) { normals(r, n); }
    #pragma unroll
    for(int i = 0; i < 4; i++) { out[i] = drawValue(v, s, group, i, r, n); }
}

// FixedProbability / FixedProbabilityNoAutapse (include/genn/genn/initSparseConnectivitySnippet.h:170-187, 208-230), one row
// by one wave64.  Lane l owns post indices [l*slice, (l+1)*slice) and walks them with the snippet's geometric skips
// `prev += 1 + (int)(log(u) * probLogRecip)`; the walk is memoryless, so restarting it at a slice boundary, or stepping over
// the diagonal without emitting (the snippet redraws instead), leaves the distribution unchanged.  First pass: counts, summed
// across the wave; second pass (same draws): sink(position in the row, postsynaptic index), ascending.  Returns the row length.
template<typename Sink>
__device__ __forceinline__ uint32_t fixedProbabilityRow(uint32_t row, uint32_t numPost, float probLogRecip, bool noAutapse, const Stream &s,
                                                        uint32_t lane, Sink sink)
{
    const uint32_t slice = (numPost + WAVE - 1) / WAVE;
    const uint32_t begin = min(numPost, lane * slice), end = min(numPost, begin + slice);
    uint32_t offset = 0, total = 0;
    for(int pass = 0; pass < 2; pass++) {
        uint32_t count = 0, draw = 0;
        long long j = (long long)begin - 1;
        Words r;
        while(true) {
            if((draw & 3u) == 0) { r = s.at(((unsigned long long)row << 32) | (draw >> 2), lane); }
            const float skip = logf(uniformOpen(r.w[draw & 3u])) * probLogRecip;
            draw++;
            if(skip >= (float)(end - begin)) { break; }
            j += 1 + (int)skip;
            if(j >= (long long)end) { break; }
            if(noAutapse && j == (long long)row) { continue; }
            if(pass == 1) { sink(offset + count, (uint32_t)j); }
            count++;
        }
        if(pass == 0) {
            const uint32_t inclusive = waveInclusiveScan(count, (int)lane);
            offset = inclusive - count;
            total = __shfl(inclusive, WAVE - 1, WAVE);
        }
    }
    return total;
}

// FixedNumberPostWithReplacement / FixedNumberTotalWithReplacement (:242-276, 292-370), one row of n targets by one wave64.
// The snippet's loop `x += (1 - x) * (1 - pow(u, 1/c))` for c = n..1 draws the n order statistics of n uniforms in ascending
// order.  The same joint law is S_k / S_{n+1} with S the prefix sums of n+1 unit exponentials, which a wave computes 256 draws at a
// time with a scan: first the total, then — regenerating the same draws — the normalised prefix sums.  Draws 0..n: spacing k ends
// at target k, spacing n is the gap between the largest target and 1; a lane takes the four draws of one generator call.
// sink(k, post[4]) receives targets k..k+3 of the row (those below n are valid).
template<typename Sink>
__device__ __forceinline__ void fixedNumberPostRow(uint32_t row, uint32_t numPost, uint32_t n, const Stream &s, uint32_t lane, Sink sink)
{
    if(n < 4 * WAVE) {
        // a single round of draws: nothing to regenerate, the spacings stay in registers while the total is formed
        const uint32_t k = 4 * lane;
        const Words r = s.at(((unsigned long long)row << 32) | (k >> 2), 0);
        double prefix[4];
        double sum = 0.0;
        #pragma unroll
        for(int i = 0; i < 4; i++) {
            sum += (k + i <= n) ? (double)-logf(uniformOpen(r.w[i])) : 0.0;
            prefix[i] = sum;
        }
        const double inclusive = waveInclusiveScan(sum, (int)lane);
        const double scale = (double)numPost / (0.0 + __shfl(inclusive, WAVE - 1, WAVE));
        if(k < n) {
            const double before = 0.0 + (inclusive - sum);
            uint32_t post[4];
            #pragma unroll
            for(int i = 0; i < 4; i++) { post[i] = min((uint32_t)((before + prefix[i]) * scale), numPost - 1); }
            sink(k, post);
        }
        return;
    }
    double scale = 0.0;
    for(int pass = 0; pass < 2; pass++) {
        double carry = 0.0;
        for(uint32_t base = 0; base <= n; base += 4 * WAVE) {
            const uint32_t k = base + 4 * lane;
            const Words r = s.at(((unsigned long long)row << 32) | (k >> 2), 0);
            double prefix[4];
            double sum = 0.0;
            #pragma unroll
            for(int i = 0; i < 4; i++) {
                sum += (k + i <= n) ? (double)-logf(uniformOpen(r.w[i])) : 0.0;
                prefix[i] = sum;
            }
            const double inclusive = waveInclusiveScan(sum, (int)lane);
            const double before = carry + (inclusive - sum);
            if(pass == 1 && k < n) {
                uint32_t post[4];
                #pragma unroll
                for(int i = 0; i < 4; i++) { post[i] = min((uint32_t)((before + prefix[i]) * scale), numPost - 1); }
                sink(k, post);
            }
            carry += __shfl(inclusive, WAVE - 1, WAVE);
        }
        scale = (double)numPost / carry;
    }
}

// The same row by the BLOCK_WAVES wavefronts of one work-group: wave w takes rounds w, w + BLOCK_WAVES, ... of 256 draws.  The
// totals of the rounds go through `roundTotal` (LDS, one double per round, at most maxRounds), and every wave then adds them
// up in round order — the additions, and so every bit of the result, are those of the one-wave version above.
// Call with all threads of the block; returns false (nothing done) if the row has more rounds than maxRounds.
template<uint32_t BLOCK_WAVES, typename Sink>
__device__ __forceinline__ bool fixedNumberPostRowBlock(uint32_t row, uint32_t numPost, uint32_t n, const Stream &s, uint32_t lane, uint32_t wave,
                                                        double *roundTotal, uint32_t maxRounds, Sink sink)
{
    const uint32_t rounds = n / (4 * WAVE) + 1;          // draws 0..n
    if(rounds > maxRounds) { return false; }
    if(rounds <= BLOCK_WAVES) {
        // at most one round per wave: its spacings stay in registers while the totals are exchanged
        const uint32_t round = wave;
        const uint32_t k = round * 4 * WAVE + 4 * lane;
        double prefix[4] = {0.0, 0.0, 0.0, 0.0};
        double sum = 0.0, inclusive = 0.0;
        if(round < rounds) {
            const Words r = s.at(((unsigned long long)row << 32) | (k >> 2), 0);
            #pragma unroll
            for(int i = 0; i < 4; i++) {
                sum += (k + i <= n) ? (double)-logf(uniformOpen(r.w[i])) : 0.0;
                prefix[i] = sum;
            }
            inclusive = waveInclusiveScan(sum, (int)lane);
            if(lane == WAVE - 1) { roundTotal[round] = inclusive; }
        }
        __syncthreads();
        if(round < rounds && k < n) {
            double total = 0.0, carry = 0.0;
            for(uint32_t q = 0; q < rounds; q++) {
                if(q == round) { carry = total; }
                total += roundTotal[q];
            }
            const double scale = (double)numPost / total;
            const double before = carry + (inclusive - sum);
            uint32_t post[4];
            #pragma unroll
            for(int i = 0; i < 4; i++) { post[i] = min((uint32_t)((before + prefix[i]) * scale), numPost - 1); }
            sink(k, post);
        }
        __syncthreads();
        return true;
    }
    for(int pass = 0; pass < 2; pass++) {
        double scale = 0.0;
        if(pass == 1) {
            __syncthreads();
            double total = 0.0;
            for(uint32_t r = 0; r < rounds; r++) { total += roundTotal[r]; }
            scale = (double)numPost / total;
        }
        for(uint32_t round = wave; round < rounds; round += BLOCK_WAVES) {
            const uint32_t k = round * 4 * WAVE + 4 * lane;
            const Words r = s.at(((unsigned long long)row << 32) | (k >> 2), 0);
            double prefix[4];
            double sum = 0.0;
            #pragma unroll
            for(int i = 0; i < 4; i++) {
                sum += (k + i <= n) ? (double)-logf(uniformOpen(r.w[i])) : 0.0;
                prefix[i] = sum;
            }
            const double inclusive = waveInclusiveScan(sum, (int)lane);
            if(pass == 0) {
                if(lane == WAVE - 1) { roundTotal[round] = inclusive; }
            }
            else if(k < n) {
                double carry = 0.0;
                for(uint32_t q = 0; q < round; q++) { carry += roundTotal[q]; }
                const double before = carry + (inclusive - sum);
                uint32_t post[4];
                #pragma unroll
                for(int i = 0; i < 4; i++) { post[i] = min((uint32_t)((before + prefix[i]) * scale), numPost - 1); }
                sink(k, post);
            }
        }
    }
    __syncthreads();            // roundTotal is reused by the next row
    return true;
}
}   // namespace gennmi_rows

#endif
