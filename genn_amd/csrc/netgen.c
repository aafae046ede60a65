/* Deterministic synthetic-input generator (host side, multi-threaded).
 *
 * Same counter-based stream definition as genn_amd/rng.py: word(seed, stream, ctr) =
 * mix(mix(seed*GOLDEN + stream*STREAM_MULT + ctr) + GOLDEN) with SplitMix64's finaliser; uniforms
 * take the top 24 bits, integers in [0,n) use multiply-shift of the top 32 bits, normals are
 * Box-Muller (cosine branch) in double.  Every element depends only on its own counter, so the
 * result does not depend on the number of threads.
 *
 * The connectivity shapes follow the reference's snippets (FixedNumberTotalWithReplacement,
 * FixedNumberPostWithReplacement, FixedProbability: include/genn/genn/initSparseConnectivitySnippet.h:170-187,
 * 242-276, 292-370) and var-init snippets (NormalClipped / NormalClippedDelay, initVarSnippet.h:161-209),
 * but draw from this generator: the reference's own seeded draws cannot be reproduced outside it.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define GOLDEN 0x9E3779B97F4A7C15ull
#define STREAM_MULT 0xD1B54A32D192ED03ull

static inline uint64_t mix(uint64_t z)
{
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}
static inline uint64_t word(uint64_t seed, uint64_t stream, uint64_t ctr)
{
    return mix(mix(seed * GOLDEN + stream * STREAM_MULT + ctr) + GOLDEN);
}
static inline double uniform01(uint64_t seed, uint64_t stream, uint64_t ctr)
{
    return (double)(word(seed, stream, ctr) >> 40) * (1.0 / 16777216.0);
}
static inline double uniform_open(uint64_t seed, uint64_t stream, uint64_t ctr)
{
    return ((double)(word(seed, stream, ctr) >> 40) + 1.0) * (1.0 / 16777216.0);
}
static inline uint32_t randint(uint64_t seed, uint64_t stream, uint64_t ctr, uint32_t n)
{
    return (uint32_t)(((word(seed, stream, ctr) >> 32) * (uint64_t)n) >> 32);
}
static inline double normal(uint64_t seed, uint64_t stream, uint64_t ctr)
{
    const double u1 = uniform_open(seed, stream, ctr);
    const double u2 = uniform01(seed, stream + 0x40000000ull, ctr);
    return sqrt(-2.0 * log(u1)) * cos(2.0 * M_PI * u2);
}

void ng_words(uint64_t seed, uint64_t stream, uint64_t start, uint64_t count, uint64_t *out)
{
    #pragma omp parallel for schedule(static)
    for(uint64_t i = 0; i < count; i++) { out[i] = word(seed, stream, start + i); }
}

/* out[i] = (float)(offset + scale * U[0,1)) */
void ng_uniform_f32(uint64_t seed, uint64_t stream, uint64_t start, uint64_t count, double scale, double offset, float *out)
{
    #pragma omp parallel for schedule(static)
    for(uint64_t i = 0; i < count; i++) { out[i] = (float)(offset + scale * uniform01(seed, stream, start + i)); }
}

void ng_normal_f32(uint64_t seed, uint64_t stream, uint64_t start, uint64_t count, double mean, double sd, float *out)
{
    #pragma omp parallel for schedule(static)
    for(uint64_t i = 0; i < count; i++) { out[i] = (float)(mean + sd * normal(seed, stream, start + i)); }
}

static int cmp_u32(const void *a, const void *b)
{
    const uint32_t x = *(const uint32_t*)a, y = *(const uint32_t*)b;
    return (x > y) - (x < y);
}

/* FixedNumberTotalWithReplacement shape: `total` presynaptic indices are drawn uniformly (counter k of
 * `stream`), which fixes every row's length; row r then draws rowLength[r] targets uniformly with
 * replacement (stream+1, counter rowStart[r]+j) and sorts them.  rowLength must hold numPre entries.
 * Returns the longest row. */
uint32_t ng_fixed_number_total_lengths(uint64_t seed, uint64_t stream, uint32_t numPre, uint64_t total, uint32_t *rowLength)
{
    memset(rowLength, 0, (size_t)numPre * sizeof(uint32_t));
    #pragma omp parallel
    {
        uint32_t *local = (uint32_t*)calloc(numPre, sizeof(uint32_t));
        #pragma omp for schedule(static)
        for(uint64_t k = 0; k < total; k++) { local[randint(seed, stream, k, numPre)]++; }
        #pragma omp critical
        for(uint32_t r = 0; r < numPre; r++) { rowLength[r] += local[r]; }
        free(local);
    }
    uint32_t longest = 0;
    for(uint32_t r = 0; r < numPre; r++) { if(rowLength[r] > longest) { longest = rowLength[r]; } }
    return longest;
}

void ng_rows_uniform_targets(uint64_t seed, uint64_t stream, uint32_t numPre, uint32_t numPost, const uint32_t *rowLength,
                             uint32_t rowStride, uint32_t *ind)
{
    uint64_t *rowStart = (uint64_t*)malloc(((size_t)numPre + 1) * sizeof(uint64_t));
    rowStart[0] = 0;
    for(uint32_t r = 0; r < numPre; r++) { rowStart[r + 1] = rowStart[r] + rowLength[r]; }
    #pragma omp parallel for schedule(dynamic, 64)
    for(uint32_t r = 0; r < numPre; r++) {
        uint32_t *row = ind + (size_t)r * rowStride;
        const uint32_t len = rowLength[r];
        for(uint32_t j = 0; j < len; j++) { row[j] = randint(seed, stream, rowStart[r] + j, numPost); }
        qsort(row, len, sizeof(uint32_t), cmp_u32);
        for(uint32_t j = len; j < rowStride; j++) { row[j] = 0; }
    }
    free(rowStart);
}

/* FixedProbability shape: Bernoulli(p) per pair by geometric skips; row r uses counters r*budget + j.
 * Pass ind = NULL to obtain row lengths only.  Returns the longest row, or UINT32_MAX if a row
 * exhausted its counter budget. */
uint32_t ng_fixed_probability(uint64_t seed, uint64_t stream, uint32_t numPre, uint32_t numPost, double p, uint32_t budget,
                              uint32_t *rowLength, uint32_t rowStride, uint32_t *ind)
{
    const double logq = log1p(-p);
    uint32_t longest = 0;
    int overflow = 0;
    #pragma omp parallel for schedule(dynamic, 64) reduction(max:longest) reduction(|:overflow)
    for(uint32_t r = 0; r < numPre; r++) {
        int64_t pos = -1;
        uint32_t len = 0;
        for(uint32_t j = 0; ; j++) {
            if(j >= budget) { overflow = 1; break; }
            const double u = uniform_open(seed, stream, (uint64_t)r * budget + j);
            pos += (int64_t)floor(log(u) / logq) + 1;
            if(pos >= (int64_t)numPost) { break; }
            if(ind) {
                if(len < rowStride) { ind[(size_t)r * rowStride + len] = (uint32_t)pos; }
            }
            len++;
        }
        if(ind) { for(uint32_t j = len; j < rowStride; j++) { ind[(size_t)r * rowStride + j] = 0; } }
        rowLength[r] = len;
        if(len > longest) { longest = len; }
    }
    return overflow ? 0xFFFFFFFFu : longest;
}

/* Per-synapse values over the valid entries of a ragged matrix; synapse (r, j) uses counter
 * rowStart[r] + j, retry number a of the clipped normal uses that counter + a*total. */
static void row_starts(uint32_t numPre, const uint32_t *rowLength, uint64_t *rowStart)
{
    rowStart[0] = 0;
    for(uint32_t r = 0; r < numPre; r++) { rowStart[r + 1] = rowStart[r] + rowLength[r]; }
}

static inline double clipped(uint64_t seed, uint64_t stream, uint64_t ctr, uint64_t total, double mean, double sd, double lo, double hi)
{
    for(uint64_t a = 0; ; a++) {
        const double v = mean + sd * normal(seed, stream, ctr + a * total);
        if(v <= hi && v >= lo) { return v; }
    }
}

void ng_rows_clipped_normal_f32(uint64_t seed, uint64_t stream, uint32_t numPre, const uint32_t *rowLength, uint32_t rowStride,
                                double mean, double sd, double lo, double hi, float *out)
{
    uint64_t *rowStart = (uint64_t*)malloc(((size_t)numPre + 1) * sizeof(uint64_t));
    row_starts(numPre, rowLength, rowStart);
    const uint64_t total = rowStart[numPre];
    #pragma omp parallel for schedule(dynamic, 64)
    for(uint32_t r = 0; r < numPre; r++) {
        float *row = out + (size_t)r * rowStride;
        for(uint32_t j = 0; j < rowStride; j++) {
            row[j] = (j < rowLength[r]) ? (float)clipped(seed, stream, rowStart[r] + j, total, mean, sd, lo, hi) : 0.0f;
        }
    }
    free(rowStart);
}

/* NormalClippedDelay: value = rint(clipped normal in timesteps), computed in fp32 like the snippet */
void ng_rows_clipped_normal_delay_u8(uint64_t seed, uint64_t stream, uint32_t numPre, const uint32_t *rowLength, uint32_t rowStride,
                                     double mean, double sd, double lo, double hi, uint8_t *out)
{
    uint64_t *rowStart = (uint64_t*)malloc(((size_t)numPre + 1) * sizeof(uint64_t));
    row_starts(numPre, rowLength, rowStart);
    const uint64_t total = rowStart[numPre];
    #pragma omp parallel for schedule(dynamic, 64)
    for(uint32_t r = 0; r < numPre; r++) {
        uint8_t *row = out + (size_t)r * rowStride;
        for(uint32_t j = 0; j < rowStride; j++) {
            row[j] = (j < rowLength[r]) ? (uint8_t)rintf((float)clipped(seed, stream, rowStart[r] + j, total, mean, sd, lo, hi)) : 0;
        }
    }
    free(rowStart);
}

/* g[r][j] = offset[r >= split] + scale[r >= split] * U[0,1): two row classes (excitatory / inhibitory sources) */
void ng_rows_uniform_f32(uint64_t seed, uint64_t stream, uint32_t numPre, const uint32_t *rowLength, uint32_t rowStride,
                         uint32_t split, double scale0, double offset0, double scale1, double offset1, float *out)
{
    uint64_t *rowStart = (uint64_t*)malloc(((size_t)numPre + 1) * sizeof(uint64_t));
    row_starts(numPre, rowLength, rowStart);
    #pragma omp parallel for schedule(dynamic, 64)
    for(uint32_t r = 0; r < numPre; r++) {
        float *row = out + (size_t)r * rowStride;
        const double sc = (r < split) ? scale0 : scale1, of = (r < split) ? offset0 : offset1;
        for(uint32_t j = 0; j < rowStride; j++) {
            row[j] = (j < rowLength[r]) ? (float)(of + sc * uniform01(seed, stream, rowStart[r] + j)) : 0.0f;
        }
    }
    free(rowStart);
}
