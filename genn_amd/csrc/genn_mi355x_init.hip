// On-device initialisation for the MI355X (gfx950) device layer: the reference's built-in
// connectivity snippets (include/genn/genn/initSparseConnectivitySnippet.h:107-330) and value
// snippets (include/genn/genn/initVarSnippet.h:87-262), which its GPU backends run inside
// initializeKernel / initializeSparseKernel (src/genn/genn/code_generator/backendSIMT.cc:1482-1779).
//
// The reference gives every thread a hiprand Philox state and lets one thread walk one row
// (src/genn/backends/hip/backend.cc:32-50); the draws a given synapse sees therefore depend on the
// backend, and the reference's own tests only ask for the right distribution
// (tests/features/test_connect_init.py, test_rng.py).  Here every draw is a pure function of
// (seed, stream, row or element, draw number) through Philox4x32-10, so a result does not depend on
// the launch geometry, and a wavefront can generate a row twice (count, then write) without storing it:
//
//   * a row belongs to one wave64, so the row's `ind` entries leave the wave as whole cache lines;
//   * FixedProbability: the geometric-skip walk of the snippet runs independently inside each lane's
//     slice of the row (Bernoulli trials of different pairs are independent), lane counts are
//     prefix-summed across the wave;
//   * FixedNumber*WithReplacement: the snippet draws ascending targets one after the other from the
//     first order statistic of what is left; the same joint distribution — sorted uniforms — is
//     produced in parallel as normalised prefix sums of n+1 exponential spacings;
//   * value snippets stream: one Philox call per four elements, 16-byte stores.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cmath>
#include <string>

#include "genn_mi355x.h"
#include "genn_mi355x_rows.h"

namespace gennmi_detail
{
int fail(int code, const std::string &msg);
void noteDeviceWrite(const void *dev, size_t bytes);     // lets runners that hold copies of weights refresh them
int flushQueuedSteps();                                  // steps a runner has queued run before this library writes device memory
}

namespace
{
using namespace gennmi_rows;
constexpr int BLOCK = 256;

#define HIP_TRY(expr)                                                                                          \
    do {                                                                                                       \
        hipError_t e_ = (expr);                                                                                \
        if(e_ != hipSuccess) {                                                                                 \
            return gennmi_detail::fail(GENNMI_EHIP, std::string(#expr) + ": " + hipGetErrorString(e_));       \
        }                                                                                                      \
    } while(0)

template<typename T> struct Quad;
template<> struct Quad<float> { typedef float4 type; };
template<> struct Quad<uint32_t> { typedef uint4 type; };
template<> struct Quad<int32_t> { typedef int4 type; };
template<> struct Quad<uint16_t> { typedef ushort4 type; };
template<> struct Quad<uint8_t> { typedef uchar4 type; };

// Marsaglia & Tsang (2000) for shape >= 1; shape < 1 through gamma(a + 1) * u^(1/a)
__device__ float gammaDraw(const Stream &s, unsigned long long element, float a)
{
    const float boost = (a < 1.0f) ? 1.0f : 0.0f;
    const float d = (a + boost) - (1.0f / 3.0f);
    const float c = 1.0f / sqrtf(9.0f * d);
    for(uint32_t attempt = 0; ; attempt++) {
        const Words r = s.at(element, attempt);
        float n[4];
        normals(r, n);
        // words 0 and 1 give the normal, word 3 the acceptance uniform, word 2 the uniform of the shape < 1 correction
        const float x = n[0];
        float v = 1.0f + c * x;
        if(v <= 0.0f) { continue; }
        v = v * v * v;
        const float u = uniformOpen(r.w[3]);
        if(u < 1.0f - 0.0331f * (x * x) * (x * x) || logf(u) < 0.5f * x * x + d * (1.0f - v + logf(v))) {
            float g = d * v;
            if(boost != 0.0f) { g *= powf(uniformOpen(r.w[2]), 1.0f / a); }
            return g;
        }
    }
}

// Binomial(n, p) by inversion of the CDF from k = 0 (Kachitvichyanukul & Schmeiser's BINV recurrence), applied to
// slices of n short enough that (1-p)^slice stays a normal double; the slices' counts add up
__device__ uint32_t binomialDraw(const Stream &s, unsigned long long element, uint32_t n, double p)
{
    if(p <= 0.0 || n == 0) { return 0; }
    if(p >= 1.0) { return n; }
    const bool flip = p > 0.5;
    const double pp = flip ? 1.0 - p : p;
    const double logQ = log1p(-pp);
    const uint32_t maxSlice = (uint32_t)fmin(4.0e9, fmax(1.0, floor(-600.0 / logQ)));
    const double ratio = pp / (1.0 - pp);
    uint32_t total = 0, done = 0, call = 0;
    while(done < n) {
        const uint32_t m = min(maxSlice, n - done);
        const Words r = s.at(element, call++);
        double u = ((double)r.w[0] * 4294967296.0 + (double)r.w[1] + 0.5) * (1.0 / 18446744073709551616.0);
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

template<typename T>
__global__ __launch_bounds__(BLOCK)
void initVarKernel(T *out, unsigned long long count, VarInit v, Stream s)
{
    typedef typename Quad<T>::type Q;
    const unsigned long long groups = (count + 3) / 4;
    for(unsigned long long g = (unsigned long long)blockIdx.x * BLOCK + threadIdx.x; g < groups; g += (unsigned long long)gridDim.x * BLOCK) {
        T value[4];
        if(v.snippet == GENNMI_INIT_GAMMA || v.snippet == GENNMI_INIT_BINOMIAL) {
            for(int k = 0; k < 4; k++) {
                const unsigned long long e = g * 4 + k;
                if(e < count) {
                    value[k] = (v.snippet == GENNMI_INIT_GAMMA) ? (T)(v.p[1] * gammaDraw(s, e, v.p[0]))
                                                               : (T)binomialDraw(s, e, (uint32_t)v.p64[0], v.p64[1]);
                }
            }
        }
        else {
            const Words r = s.at(g, 0);
            float n[4] = {0.0f, 0.0f, 0.0f, 0.0f};
            if(v.snippet == GENNMI_INIT_NORMAL || v.snippet == GENNMI_INIT_NORMAL_CLIPPED || v.snippet == GENNMI_INIT_NORMAL_CLIPPED_DELAY) {
                normals(r, n);
            }
            #pragma unroll
            for(int k = 0; k < 4; k++) { value[k] = (T)drawValue(v, s, g, k, r, n); }
        }
        if(g * 4 + 3 < count) {
            Q q;
            q.x = value[0]; q.y = value[1]; q.z = value[2]; q.w = value[3];
            *reinterpret_cast<Q*>(out + g * 4) = q;
        }
        else {
            for(int k = 0; k < 4 && g * 4 + k < count; k++) { out[g * 4 + k] = value[k]; }
        }
    }
}

__global__ __launch_bounds__(BLOCK)
void randomWordsKernel(uint32_t *out, unsigned long long count, Stream s)
{
    const unsigned long long groups = (count + 3) / 4;
    for(unsigned long long g = (unsigned long long)blockIdx.x * BLOCK + threadIdx.x; g < groups; g += (unsigned long long)gridDim.x * BLOCK) {
        const Words r = s.at(g, 0);
        for(int k = 0; k < 4 && g * 4 + k < count; k++) { out[g * 4 + k] = r.w[k]; }
    }
}

__device__ uint32_t g_rowOverflow;      // rows that wanted more entries than rowStride, last connectivity launch

// FixedProbability / FixedProbabilityNoAutapse: one row per wave64, generated by fixedProbabilityRow() and stored
__global__ __launch_bounds__(BLOCK)
void fixedProbabilityKernel(uint32_t numPre, uint32_t numPost, uint32_t rowStride, float probLogRecip, int noAutapse, Stream s,
                            uint32_t *rowLength, uint32_t *ind)
{
    const uint32_t lane = threadIdx.x & (WAVE - 1);
    const uint32_t row = blockIdx.x * (BLOCK / WAVE) + threadIdx.x / WAVE;
    if(row >= numPre) { return; }
    uint32_t *rowInd = ind + (size_t)row * rowStride;
    const uint32_t total = fixedProbabilityRow(row, numPost, probLogRecip, noAutapse != 0, s, lane,
                                               [&](uint32_t k, uint32_t post) { if(k < rowStride) { rowInd[k] = post; } });
    if(lane == 0) {
        rowLength[row] = min(total, rowStride);
        if(total > rowStride) { atomicAdd(&g_rowOverflow, 1u); }
    }
}

// FixedNumberPostWithReplacement / FixedNumberTotalWithReplacement: one row per wave64, generated by fixedNumberPostRow() and
// stored 1 KiB of the row at a time
__global__ __launch_bounds__(BLOCK)
void fixedNumberPostKernel(uint32_t numPre, uint32_t numPost, uint32_t rowStride, uint32_t num, const uint32_t *rowLengthIn, Stream s,
                           uint32_t *rowLength, uint32_t *ind)
{
    const uint32_t lane = threadIdx.x & (WAVE - 1);
    const uint32_t row = blockIdx.x * (BLOCK / WAVE) + threadIdx.x / WAVE;
    if(row >= numPre) { return; }
    uint32_t n = rowLengthIn ? rowLengthIn[row] : num;
    if(n > rowStride) {
        if(lane == 0) { atomicAdd(&g_rowOverflow, 1u); }
        n = rowStride;
    }
    uint32_t *rowInd = ind + (size_t)row * rowStride;
    const bool vectorStores = ((rowStride & 3u) == 0) && (((uintptr_t)ind & 15u) == 0);
    fixedNumberPostRow(row, numPost, n, s, lane, [&](uint32_t k, const uint32_t post[4]) {
        if(vectorStores && k + 3 < n) {
            *reinterpret_cast<uint4*>(rowInd + k) = make_uint4(post[0], post[1], post[2], post[3]);
        }
        else {
            for(int i = 0; i < 4 && k + i < n; i++) { rowInd[k + i] = post[i]; }
        }
    });
    if(lane == 0) { rowLength[row] = n; }
}

// OneToOne (initSparseConnectivitySnippet.h:107-118)
__global__ void oneToOneKernel(uint32_t numPre, uint32_t numPost, uint32_t rowStride, uint32_t *rowLength, uint32_t *ind)
{
    const uint32_t row = blockIdx.x * blockDim.x + threadIdx.x;
    if(row < numPre) {
        const bool valid = row < numPost;
        rowLength[row] = valid ? 1u : 0u;
        if(valid) { ind[(size_t)row * rowStride] = row; }
    }
}

// FixedNumberPreWithReplacement (initSparseConnectivitySnippet.h:380-410): every postsynaptic neuron draws `num` sources,
// idPre = gennrand() % num_pre, and each draw appends the neuron to its source's row.  A thread makes four draws of one
// column (one generator call); rows are appended to through an atomic counter, in arbitrary order ...
__global__ __launch_bounds__(BLOCK)
void fixedNumberPreScatterKernel(uint32_t numPre, uint32_t numPost, uint32_t rowStride, uint32_t num, Stream s, uint32_t *rowLength, uint32_t *ind)
{
    const uint32_t groupsPerColumn = (num + 3) / 4;
    const unsigned long long item = (unsigned long long)blockIdx.x * BLOCK + threadIdx.x;
    if(item >= (unsigned long long)numPost * groupsPerColumn) { return; }
    const uint32_t column = (uint32_t)(item / groupsPerColumn), group = (uint32_t)(item - (unsigned long long)column * groupsPerColumn);
    const Words r = s.at(item, 0);
    #pragma unroll
    for(int k = 0; k < 4; k++) {
        if(group * 4 + k >= num) { break; }
        const uint32_t idPre = r.w[k] % numPre;
        const uint32_t position = atomicAdd(&rowLength[idPre], 1u);
        if(position < rowStride) { ind[(size_t)idPre * rowStride + position] = column; }
        else if(position == rowStride) { atomicAdd(&g_rowOverflow, 1u); }
    }
}
// ... and then sorted (one work-group per row, bitonic network in LDS over the next power of two), so that rows come out
// ascending like those of every other generator here, whatever order the appends happened in
__global__ __launch_bounds__(BLOCK)
void rowSortKernel(uint32_t rowStride, uint32_t *rowLength, uint32_t *ind, uint32_t capacity)
{
    extern __shared__ uint32_t shRow[];
    const uint32_t row = blockIdx.x;
    const uint32_t length = min(rowLength[row], rowStride);
    if(threadIdx.x == 0) { rowLength[row] = length; }
    if(length < 2) { return; }
    uint32_t n = 2;
    while(n < length) { n <<= 1; }
    (void)capacity;
    uint32_t *entries = ind + (size_t)row * rowStride;
    for(uint32_t i = threadIdx.x; i < n; i += BLOCK) { shRow[i] = (i < length) ? entries[i] : 0xFFFFFFFFu; }
    __syncthreads();
    for(uint32_t k = 2; k <= n; k <<= 1) {
        for(uint32_t j = k >> 1; j > 0; j >>= 1) {
            for(uint32_t i = threadIdx.x; i < n; i += BLOCK) {
                const uint32_t partner = i ^ j;
                if(partner > i) {
                    const uint32_t a = shRow[i], b = shRow[partner];
                    const bool ascending = ((i & k) == 0);
                    if((a > b) == ascending) { shRow[i] = b; shRow[partner] = a; }
                }
            }
            __syncthreads();
        }
    }
    for(uint32_t i = threadIdx.x; i < length; i += BLOCK) { entries[i] = shRow[i]; }
}

// Conv2D as SPARSE connectivity (initSparseConnectivitySnippet.h:438-497): the snippet's row build code, one thread per
// presynaptic neuron; targets come out ascending (output row, column, channel).  With `kernel` and `g`, every synapse's weight
// is the kernel entry its (kernel row, kernel column, input channel, output channel) names — InitVarSnippet::Kernel
// (initVarSnippet.h:100-108) over the snippet's kernel size {kh, kw, ic, oc}.
struct Conv2DParams { int kh, kw, sh, sw, padh, padw, ih, iw, ic, oh, ow, oc; };
__global__ __launch_bounds__(BLOCK)
void conv2dSparseKernel(Conv2DParams c, uint32_t rowStride, uint32_t *rowLength, uint32_t *ind, const float *kernel, float *g)
{
    const uint32_t idPre = blockIdx.x * BLOCK + threadIdx.x;
    if(idPre >= (uint32_t)(c.ih * c.iw * c.ic)) { return; }
    const int inRow = ((int)idPre / c.ic) / c.iw, inCol = ((int)idPre / c.ic) % c.iw, inChan = (int)idPre % c.ic;
    const int maxOutRow = min(c.oh, max(0, 1 + ((inRow + c.padh) / c.sh)));
    const int minOutCol = min(c.ow, max(0, 1 + (int)floorf((float)(inCol + c.padw - c.kw) / (float)c.sw)));
    const int maxOutCol = min(c.ow, max(0, 1 + ((inCol + c.padw) / c.sw)));
    int outRow = min(c.oh, max(0, 1 + (int)floorf((float)(inRow + c.padh - c.kh) / (float)c.sh)));
    uint32_t length = 0;
    for(; outRow < maxOutRow; outRow++) {
        const int kernRow = inRow - ((outRow * c.sh) - c.padh);
        for(int outCol = minOutCol; outCol < maxOutCol; outCol++) {
            const int kernCol = inCol - ((outCol * c.sw) - c.padw);
            for(int outChan = 0; outChan < c.oc; outChan++) {
                if(length < rowStride) {
                    const size_t idSyn = (size_t)idPre * rowStride + length;
                    ind[idSyn] = (uint32_t)((outRow * c.ow * c.oc) + (outCol * c.oc) + outChan);
                    if(g) { g[idSyn] = kernel[((size_t)(kernRow * c.kw + kernCol) * c.ic + inChan) * c.oc + outChan]; }
                }
                length++;
            }
        }
    }
    if(length > rowStride) { atomicAdd(&g_rowOverflow, 1u); length = rowStride; }
    rowLength[idPre] = length;
}

Stream makeStream(uint64_t seed, uint32_t stream) { return Stream{(uint32_t)seed, (uint32_t)(seed >> 32), stream}; }

int finishConnectivity(uint32_t *overflowRows)
{
    HIP_TRY(hipGetLastError());
    uint32_t overflow = 0;
    HIP_TRY(hipMemcpyFromSymbol(&overflow, HIP_SYMBOL(g_rowOverflow), sizeof(uint32_t)));
    if(overflowRows) { *overflowRows = overflow; }
    if(overflow) {
        return gennmi_detail::fail(GENNMI_EINVAL, std::to_string(overflow) + " row(s) drew more synapses than rowStride holds; the rows were truncated");
    }
    return GENNMI_OK;
}

int clearOverflow()
{
    const uint32_t zero = 0;
    HIP_TRY(hipMemcpyToSymbol(HIP_SYMBOL(g_rowOverflow), &zero, sizeof(uint32_t)));
    return GENNMI_OK;
}

template<typename T>
int launchInitVar(void *dev, size_t count, const VarInit &v, const Stream &s)
{
    const unsigned long long groups = (count + 3) / 4;
    const unsigned int blocks = (unsigned int)std::min<unsigned long long>((groups + BLOCK - 1) / BLOCK, 256ull * 32ull);
    hipLaunchKernelGGL(initVarKernel<T>, dim3(blocks), dim3(BLOCK), 0, 0, (T*)dev, (unsigned long long)count, v, s);
    HIP_TRY(hipGetLastError());
    return GENNMI_OK;
}
}   // anonymous namespace

extern "C" {

int gennmi_philox4x32(const uint32_t counter[4], const uint32_t key[2], uint32_t out[4])
{
    const Words r = philox4x32(counter[0], counter[1], counter[2], counter[3], key[0], key[1]);
    for(int k = 0; k < 4; k++) { out[k] = r.w[k]; }
    return GENNMI_OK;
}

int gennmi_init_random_words(uint32_t *dev, size_t count, uint64_t seed, uint32_t stream)
{
    { const int rcFlush = gennmi_detail::flushQueuedSteps(); if(rcFlush) { return rcFlush; } }
    if(count == 0) { return GENNMI_OK; }
    const unsigned long long groups = (count + 3) / 4;
    const unsigned int blocks = (unsigned int)std::min<unsigned long long>((groups + BLOCK - 1) / BLOCK, 256ull * 32ull);
    hipLaunchKernelGGL(randomWordsKernel, dim3(blocks), dim3(BLOCK), 0, 0, dev, (unsigned long long)count, makeStream(seed, stream));
    HIP_TRY(hipGetLastError());
    return GENNMI_OK;
}

int gennmi_init_var(void *dev, uint32_t elementType, size_t count, uint32_t snippet, const double params[4], uint64_t seed, uint32_t stream)
{
    { const int rcFlush = gennmi_detail::flushQueuedSteps(); if(rcFlush) { return rcFlush; } }
    if(count == 0) { return GENNMI_OK; }
    if(snippet > GENNMI_INIT_BINOMIAL) { return gennmi_detail::fail(GENNMI_EUNSUPPORTED, "unknown value-initialisation snippet"); }
    if((uintptr_t)dev % 16) { return gennmi_detail::fail(GENNMI_EINVAL, "array to initialise is not 16-byte aligned"); }
    VarInit v;
    v.snippet = snippet;
    for(int k = 0; k < 4; k++) { v.p[k] = (float)params[k]; }
    v.p64[0] = params[0];
    v.p64[1] = params[1];
    if((snippet == GENNMI_INIT_NORMAL_CLIPPED || snippet == GENNMI_INIT_NORMAL_CLIPPED_DELAY) && !(v.p[2] < v.p[3])) {
        return gennmi_detail::fail(GENNMI_EINVAL, "clipped normal needs min < max");
    }
    if(snippet == GENNMI_INIT_GAMMA && !(v.p[0] > 0.0f)) { return gennmi_detail::fail(GENNMI_EINVAL, "gamma shape must be positive"); }
    if(snippet == GENNMI_INIT_BINOMIAL && !(params[0] >= 0.0 && params[0] < 4294967296.0 && params[1] >= 0.0 && params[1] <= 1.0)) {
        return gennmi_detail::fail(GENNMI_EINVAL, "binomial needs 0 <= n < 2^32 and 0 <= p <= 1");
    }
    const Stream s = makeStream(seed, stream);
    gennmi_detail::noteDeviceWrite(dev, count * 4);
    switch(elementType) {
    case GENNMI_TYPE_F32: return launchInitVar<float>(dev, count, v, s);
    case GENNMI_TYPE_U32: return launchInitVar<uint32_t>(dev, count, v, s);
    case GENNMI_TYPE_I32: return launchInitVar<int32_t>(dev, count, v, s);
    case GENNMI_TYPE_U16: return launchInitVar<uint16_t>(dev, count, v, s);
    case GENNMI_TYPE_U8: return launchInitVar<uint8_t>(dev, count, v, s);
    default: return gennmi_detail::fail(GENNMI_EUNSUPPORTED, "unknown element type");
    }
}

int gennmi_init_sparse_fixed_probability(uint32_t numPre, uint32_t numPost, uint32_t rowStride, double prob, int noAutapse,
                                         uint64_t seed, uint32_t stream, uint32_t *rowLength, uint32_t *ind, uint32_t *overflowRows)
{
    { const int rcFlush = gennmi_detail::flushQueuedSteps(); if(rcFlush) { return rcFlush; } }
    if(!(prob >= 0.0 && prob <= 1.0)) { return gennmi_detail::fail(GENNMI_EINVAL, "connection probability outside [0, 1]"); }
    if(numPre == 0 || numPost == 0 || rowStride == 0) { return gennmi_detail::fail(GENNMI_EINVAL, "empty matrix"); }
    if(numPost > 0x7fffffffu || rowStride > 0x7fffffffu) { return gennmi_detail::fail(GENNMI_EINVAL, "more than 2^31-1 postsynaptic neurons or row entries"); }
    if(int rc = clearOverflow()) { return rc; }
    // probLogRecip = 1 / log(1 - prob) as the snippet's derived parameter; prob = 0 gives -inf (every skip leaves the row),
    // prob = 1 gives -0 (every skip is 0: all pairs connect)
    const float probLogRecip = (prob == 0.0) ? -INFINITY : (float)(1.0 / std::log(1.0 - prob));
    const unsigned int blocks = (numPre + (BLOCK / WAVE) - 1) / (BLOCK / WAVE);
    hipLaunchKernelGGL(fixedProbabilityKernel, dim3(blocks), dim3(BLOCK), 0, 0, numPre, numPost, rowStride, probLogRecip, noAutapse,
                       makeStream(seed, stream), rowLength, ind);
    return finishConnectivity(overflowRows);
}

int gennmi_init_sparse_fixed_number_post(uint32_t numPre, uint32_t numPost, uint32_t rowStride, uint32_t num, const uint32_t *rowLengthIn,
                                         uint64_t seed, uint32_t stream, uint32_t *rowLength, uint32_t *ind, uint32_t *overflowRows)
{
    { const int rcFlush = gennmi_detail::flushQueuedSteps(); if(rcFlush) { return rcFlush; } }
    if(numPre == 0 || numPost == 0 || rowStride == 0) { return gennmi_detail::fail(GENNMI_EINVAL, "empty matrix"); }
    if(!rowLengthIn && num > rowStride) { return gennmi_detail::fail(GENNMI_EINVAL, "num exceeds rowStride"); }
    if(rowStride > 0x7fffffffu) { return gennmi_detail::fail(GENNMI_EINVAL, "more than 2^31-1 row entries"); }
    if(int rc = clearOverflow()) { return rc; }
    const unsigned int blocks = (numPre + (BLOCK / WAVE) - 1) / (BLOCK / WAVE);
    hipLaunchKernelGGL(fixedNumberPostKernel, dim3(blocks), dim3(BLOCK), 0, 0, numPre, numPost, rowStride, num, rowLengthIn,
                       makeStream(seed, stream), rowLength, ind);
    return finishConnectivity(overflowRows);
}

int gennmi_init_sparse_fixed_number_pre(uint32_t numPre, uint32_t numPost, uint32_t rowStride, uint32_t num,
                                        uint64_t seed, uint32_t stream, uint32_t *rowLength, uint32_t *ind, uint32_t *overflowRows)
{
    { const int rcFlush = gennmi_detail::flushQueuedSteps(); if(rcFlush) { return rcFlush; } }
    if(numPre == 0 || numPost == 0 || rowStride == 0) { return gennmi_detail::fail(GENNMI_EINVAL, "empty matrix"); }
    if(rowStride > 16384) { return gennmi_detail::fail(GENNMI_EUNSUPPORTED, "rows of more than 16384 entries are not sorted on the device"); }
    if(int rc = clearOverflow()) { return rc; }
    HIP_TRY(hipMemset(rowLength, 0, (size_t)numPre * sizeof(uint32_t)));
    const unsigned long long items = (unsigned long long)numPost * ((num + 3) / 4);
    if(items > 0x7fffffffull * BLOCK) { return gennmi_detail::fail(GENNMI_EINVAL, "too many draws for one launch"); }
    if(items) {
        hipLaunchKernelGGL(fixedNumberPreScatterKernel, dim3((unsigned int)((items + BLOCK - 1) / BLOCK)), dim3(BLOCK), 0, 0, numPre, numPost, rowStride, num,
                           makeStream(seed, stream), rowLength, ind);
    }
    uint32_t capacity = 2;
    while(capacity < rowStride) { capacity <<= 1; }
    if(capacity * sizeof(uint32_t) > 48 * 1024) {
        HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void*>(rowSortKernel), hipFuncAttributeMaxDynamicSharedMemorySize, (int)(capacity * sizeof(uint32_t))));
    }
    hipLaunchKernelGGL(rowSortKernel, dim3(numPre), dim3(BLOCK), capacity * sizeof(uint32_t), 0, rowStride, rowLength, ind, capacity);
    return finishConnectivity(overflowRows);
}

int gennmi_init_sparse_conv2d(const int32_t conv[12], uint32_t rowStride, uint32_t *rowLength, uint32_t *ind, const float *kernel, float *g,
                              uint32_t *overflowRows)
{
    { const int rcFlush = gennmi_detail::flushQueuedSteps(); if(rcFlush) { return rcFlush; } }
    if(!conv || !rowLength || !ind || rowStride == 0 || ((kernel == nullptr) != (g == nullptr))) { return gennmi_detail::fail(GENNMI_EINVAL, "init_sparse_conv2d: bad arguments"); }
    const Conv2DParams c{conv[0], conv[1], conv[2], conv[3], conv[4], conv[5], conv[6], conv[7], conv[8], conv[9], conv[10], conv[11]};
    if(c.kh <= 0 || c.kw <= 0 || c.sh <= 0 || c.sw <= 0 || c.padh < 0 || c.padw < 0 || c.ih <= 0 || c.iw <= 0 || c.ic <= 0 || c.oh <= 0 || c.ow <= 0 || c.oc <= 0) {
        return gennmi_detail::fail(GENNMI_EINVAL, "init_sparse_conv2d: sizes and strides must be positive, padding non-negative");
    }
    if((unsigned long long)c.ih * c.iw * c.ic > 0xffffffffull || (unsigned long long)c.oh * c.ow * c.oc > 0xffffffffull) {
        return gennmi_detail::fail(GENNMI_EINVAL, "init_sparse_conv2d: more than 2^32-1 neurons");
    }
    if(int rc = clearOverflow()) { return rc; }
    const uint32_t numPre = (uint32_t)(c.ih * c.iw * c.ic);
    hipLaunchKernelGGL(conv2dSparseKernel, dim3((numPre + BLOCK - 1) / BLOCK), dim3(BLOCK), 0, 0, c, rowStride, rowLength, ind, kernel, g);
    gennmi_detail::noteDeviceWrite(ind, (size_t)numPre * rowStride * sizeof(uint32_t));
    if(g) { gennmi_detail::noteDeviceWrite(g, (size_t)numPre * rowStride * sizeof(float)); }
    return finishConnectivity(overflowRows);
}

int gennmi_init_sparse_one_to_one(uint32_t numPre, uint32_t numPost, uint32_t rowStride, uint32_t *rowLength, uint32_t *ind)
{
    { const int rcFlush = gennmi_detail::flushQueuedSteps(); if(rcFlush) { return rcFlush; } }
    if(numPre == 0 || numPost == 0 || rowStride == 0) { return gennmi_detail::fail(GENNMI_EINVAL, "empty matrix"); }
    hipLaunchKernelGGL(oneToOneKernel, dim3((numPre + BLOCK - 1) / BLOCK), dim3(BLOCK), 0, 0, numPre, numPost, rowStride, rowLength, ind);
    HIP_TRY(hipGetLastError());
    return GENNMI_OK;
}

}   // extern "C"
