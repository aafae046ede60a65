/* TEST INFRASTRUCTURE — not product code.  Only tests/, __graft_entry__.smoke() and the
 * cpu_baseline leg of bench.py may load this library, and only as the checker / baseline.
 *
 * Single-threaded CPU restatement of what the reference's SingleThreadedCPU backend generates
 * for the per-timestep hot path, in plain C.  Arithmetic is fp32 with one rounding per
 * operation (build with -ffp-contract=off, no fast-math), matching the reference's generated
 * C++ which is compiled without -O / -march (src/genn/backends/single_threaded_cpu/backend.cc:1615-1635).
 * All model constants arrive already rounded to fp32 by the caller.
 *
 * Reference code each function follows (paths under the reference tree):
 *   gc_update_synapses   dendritic pointer advance   src/genn/backends/single_threaded_cpu/backend.cc:426-442,
 *                                                    src/genn/genn/code_generator/synapseUpdateGroupMerged.cc:480-483
 *                        sparse presynaptic loop     backend.cc:1884-1929, synapseUpdateGroupMerged.cc:49-217, 245-251
 *                        Toeplitz presynaptic loop   backend.cc:1788-1883, include/genn/genn/initToeplitzConnectivitySnippet.h:116-137
 *                        dense / bitmask loop        backend.cc:1985-2021 (bit gid = idPre*rowStride + idPost, most significant bit
 *                                                    first; row stride = numPost padded to 32, backend.cc:1393-1404)
 *                        presynaptic output          addToPre backend.cc:1822; consumed neuronUpdateGroupMerged.cc:148-165, 591-595
 *                        spike-like events           backend.cc:537-540 + the sparse loop with the event code of
 *                                                    include/genn/genn/weightUpdateModels.h:308-319 (StaticGraded)
 *                        postsynaptic (learnPost)    backend.cc:2029-2095
 *   gc_update_neurons    spike queue reset           src/genn/genn/code_generator/neuronUpdateGroupMerged.cc:947-975
 *                        neuron loop + op order      backend.cc:187-398, neuronUpdateGroupMerged.cc:552-773 (PSM :66-137, CS :20-55,
 *                                                    WU pre/post :333-459), spike emission backend.cc:2119-2133
 *                        event conditions            neuronUpdateGroupMerged.cc:215-330, 677-683; emission backend.cc genEmitEvent
 *                        PoissonExp source           include/genn/genn/currentSourceModels.h:100-129 (the generator behind gennrand_uniform is this
 *                                                    build's own counter-based one: parity with the reference is statistical)
 *                        model arithmetic            include/genn/genn/neuronModels.h:163-186 (Izhikevich), :220-257 (LIF), :274-286
 *                                                    (SpikeSourceArray); postsynapticModels.h:91-106 (ExpCurr), DeltaCurr;
 *                                                    currentSourceModels.h:70-77 (DC); weightUpdateModels.h:236-287;
 *                                                    trace STDP = pygenn/genn_model.py:1448-1476
 *   gc_build_remap       column view                 backend.cc:156-179
 *   gc_step              order + time                src/genn/genn/code_generator/generateRunner.cc:270-299
 *
 * Parity pins: golden vectors written by the reference's own CPU backend (tests/golden/, made
 * by tests/golden/make_golden.py through oracle/ref_driver.cc), the closed-form decode tables
 * of the reference's tests/features/test_event_propagation.py, and its Toeplitz fixtures.  The dense / bitmask loop has no
 * golden vector from the reference's backend: it is pinned by that decode table (test_event_propagation.py:237-260 holds
 * for its DENSE and BITMASK projections too) and by brute force against a matrix-vector product (tests/test_oracle_golden.py).
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

enum { GC_LIF = 0, GC_IZH = 1, GC_SSA = 2 };
enum { GC_EXPCURR = 0, GC_DELTACURR = 1 };
enum { GC_STATIC = 0, GC_STATIC_DELAY = 1, GC_STDP_TRACE = 2, GC_STATIC_GRADED = 3, GC_STATIC_REVERSE = 4, GC_STDP_ADDITIVE = 5 };
enum { GC_SPARSE = 0, GC_CONV2D = 1, GC_DENSE = 2, GC_BITMASK = 3 };
enum { GC_CS_DC = 0, GC_CS_NOISE = 1, GC_CS_POISSON_EXP = 2 };

#define GC_MAX_CHILD 16
#define GC_MAX_EVENT 4

/* one spike-like event queue of a population ("SynSpikeEvent" child): condition V > threshold */
typedef struct {
    float threshold;
    uint32_t *spkEvent, spkCntEvent;
    uint32_t *recordSpkEvent;   /* [numRec * ceil(n/32)] or NULL (runtime.cc:307-311) */
} gc_event;

typedef struct {
    int kind;            /* GC_EXPCURR / GC_DELTACURR */
    float init, expDecay;
    uint32_t maxDenDelay;   /* 0: no dendritic delay */
    float *outPost;         /* [n] */
    float *denDelay;        /* [maxDenDelay * n], slot-major */
    uint32_t denDelayPtr;
} gc_psm;

typedef struct {
    int kind;
    float amp;
    const float *noise;     /* [noiseSteps * n]: row s % noiseSteps is what the host pushes before step s */
    uint64_t noiseSteps;
    /* PoissonExp (currentSourceModels.h:100-129): state variable and derived parameters; the uniforms of neuron i in step k
     * are the words of Philox4x32-10(counter = (indexOffset + i, k, call, stream), key = seed), call = 0, 1, ... */
    float *current; float init, expDecay, expMinusLambda;
    uint64_t seed; uint32_t stream, indexOffset;
} gc_cs;

typedef struct {
    int model;
    uint32_t n;
    /* LIF: p = {Ioffset, Rmembrane, Vrest, ExpTC, Vthresh, Vreset, TauRefrac}; IZH: {a,b,c,d} */
    float p[8];
    float *v0, *v1;         /* LIF: V, RefracTime; IZH: V, U */
    uint32_t *startSpike; const uint32_t *endSpike; const float *spikeTimes;
    int numPSM; gc_psm psm[GC_MAX_CHILD];
    int numCS; gc_cs cs[GC_MAX_CHILD];
    /* fused WU pre / post trace variables (one each is all the configurations need) */
    float *preTrace, *postTrace; float preDecay, postDecay;
    float *sT;              /* spike times, allocated when a WU model reads st_pre / st_post */
    uint32_t *spk, spkCnt;  /* the queue written by the last neuron update (slot spkQuePtr of the ring below, if there is one) */
    /* axonal delay (backendBase.cc:128-162): ring of numDelaySlots queues, slot-major; spkQuePtr advances at the start of
     * every neuron update (neuronUpdateGroupMerged.cc:947-953) */
    uint32_t numDelaySlots, spkQuePtr;
    uint32_t *spkRing, *spkCntRing;
    uint32_t *recordSpk;    /* [numRec * ceil(n/32)] or NULL */
    int numEvents; gc_event events[GC_MAX_EVENT];
    /* presynaptic output of outgoing projections whose code calls addToPre ("OutSynPreOutput" children) */
    int numPreOutput; float *outPre[GC_MAX_EVENT];
} gc_pop;

typedef struct {
    int matrix, wum;
    int src, trg, psm;
    uint32_t rowStride, colStride;
    const uint32_t *rowLength, *ind; float *g; const uint8_t *d;
    uint32_t *colLength, *remap;
    float aPlus, aMinus, wMin, wMax;
    float tauPlus, tauMinus;   /* GC_STDP_ADDITIVE */
    int conv[8]; int conv_bh, conv_bw;
    uint32_t delaySteps;    /* axonal delay in timesteps: reads slot (spkQuePtr + slots - delaySteps) % slots of the source */
    const uint32_t *gp;     /* BITMASK connectivity words */
    float constantWeight;   /* StaticPulseConstantWeight (weightUpdateModels.h:202-213): used when g is NULL */
    int event; float epre, vslope;   /* StaticGraded: which of the source's event queues it reads, and its parameters */
    int preOutput;          /* GC_STATIC_REVERSE: which outPre of the source it adds to */
    uint64_t events;        /* synaptic events processed so far (bookkeeping, not in the reference) */
} gc_syn;

typedef struct {
    float dt;
    uint64_t timestep, numRec;
    int numPops, numSyns, capPops, capSyns;
    gc_pop *pops; gc_syn *syns;
} gc_net;

/* ------------------------------------------------------------------------------------------ */
gc_net *gc_create(float dt, uint64_t numRecordingTimesteps)
{
    gc_net *net = (gc_net*)calloc(1, sizeof(gc_net));
    net->dt = dt;
    net->numRec = numRecordingTimesteps;
    return net;
}

static void *gc_dup(const void *src, size_t bytes)
{
    void *p = malloc(bytes ? bytes : 1);
    if(src) { memcpy(p, src, bytes); } else { memset(p, 0, bytes); }
    return p;
}

int gc_add_pop(gc_net *net, int model, uint32_t n, const float *params, int numParams,
               const void *var0, const void *var1, const float *spikeTimes)
{
    if(net->numPops == net->capPops) {
        net->capPops = net->capPops ? net->capPops * 2 : 8;
        net->pops = (gc_pop*)realloc(net->pops, net->capPops * sizeof(gc_pop));
    }
    gc_pop *p = &net->pops[net->numPops];
    memset(p, 0, sizeof(*p));
    p->model = model; p->n = n;
    for(int i = 0; i < numParams && i < 8; i++) { p->p[i] = params[i]; }
    if(model == GC_SSA) {
        p->startSpike = (uint32_t*)gc_dup(var0, n * sizeof(uint32_t));
        p->endSpike = (const uint32_t*)gc_dup(var1, n * sizeof(uint32_t));
        p->spikeTimes = spikeTimes;     /* caller keeps it alive */
    }
    else {
        p->v0 = (float*)gc_dup(var0, n * sizeof(float));
        p->v1 = (float*)gc_dup(var1, n * sizeof(float));
    }
    p->spk = (uint32_t*)calloc(n ? n : 1, sizeof(uint32_t));
    if(net->numRec) { p->recordSpk = (uint32_t*)calloc(net->numRec * ((n + 31) / 32), sizeof(uint32_t)); }
    return net->numPops++;
}

/* numDelaySlots = longest axonal delay of the population's outgoing projections + 1 (neuronGroup.cc checkNumDelaySlots) */
void gc_set_delay_slots(gc_net *net, int pop, uint32_t numDelaySlots)
{
    gc_pop *p = &net->pops[pop];
    if(numDelaySlots > 1) {
        p->numDelaySlots = numDelaySlots;
        p->spkRing = (uint32_t*)calloc((size_t)numDelaySlots * (p->n ? p->n : 1), sizeof(uint32_t));
        p->spkCntRing = (uint32_t*)calloc(numDelaySlots, sizeof(uint32_t));
        free(p->spk);
        p->spk = p->spkRing;
    }
}

void gc_set_axonal_delay(gc_net *net, int syn, uint32_t delaySteps) { net->syns[syn].delaySteps = delaySteps; }

int gc_add_psm(gc_net *net, int pop, int kind, float init, float expDecay, uint32_t maxDenDelay)
{
    gc_pop *p = &net->pops[pop];
    if(p->numPSM == GC_MAX_CHILD) { return -1; }
    gc_psm *m = &p->psm[p->numPSM];
    m->kind = kind; m->init = init; m->expDecay = expDecay; m->maxDenDelay = maxDenDelay;
    m->outPost = (float*)calloc(p->n ? p->n : 1, sizeof(float));
    m->denDelay = maxDenDelay ? (float*)calloc((size_t)maxDenDelay * p->n, sizeof(float)) : NULL;
    m->denDelayPtr = 0;
    return p->numPSM++;
}

int gc_add_cs(gc_net *net, int pop, int kind, float amp, const float *noise, uint64_t noiseSteps)
{
    gc_pop *p = &net->pops[pop];
    if(p->numCS == GC_MAX_CHILD) { return -1; }
    p->cs[p->numCS].kind = kind; p->cs[p->numCS].amp = amp; p->cs[p->numCS].noise = noise;
    p->cs[p->numCS].noiseSteps = noiseSteps ? noiseSteps : 1;
    return p->numCS++;
}

/* Philox4x32-10 (Salmon et al., SC'11): the published round function and key schedule */
void gc_philox4x32(uint32_t c0, uint32_t c1, uint32_t c2, uint32_t c3, uint32_t k0, uint32_t k1, uint32_t out[4])
{
    for(int round = 0; round < 10; round++) {
        const uint64_t p0 = (uint64_t)0xD2511F53u * c0, p1 = (uint64_t)0xCD9E8D57u * c2;
        const uint32_t hi0 = (uint32_t)(p0 >> 32), lo0 = (uint32_t)p0, hi1 = (uint32_t)(p1 >> 32), lo1 = (uint32_t)p1;
        c0 = hi1 ^ c1 ^ k0; c1 = lo1; c2 = hi0 ^ c3 ^ k1; c3 = lo0;
        k0 += 0x9E3779B9u; k1 += 0xBB67AE85u;
    }
    out[0] = c0; out[1] = c1; out[2] = c2; out[3] = c3;
}

int gc_add_cs_poisson_exp(gc_net *net, int pop, float init, float expDecay, float expMinusLambda, uint64_t seed, uint32_t stream,
                          uint32_t indexOffset, const float *current0)
{
    gc_pop *p = &net->pops[pop];
    if(p->numCS == GC_MAX_CHILD) { return -1; }
    gc_cs *c = &p->cs[p->numCS];
    memset(c, 0, sizeof(*c));
    c->kind = GC_CS_POISSON_EXP; c->init = init; c->expDecay = expDecay; c->expMinusLambda = expMinusLambda;
    c->seed = seed; c->stream = stream; c->indexOffset = indexOffset; c->noiseSteps = 1;
    c->current = (float*)gc_dup(current0, (size_t)p->n * sizeof(float));
    return p->numCS++;
}

float *gc_cs_current(gc_net *net, int pop, int cs) { return net->pops[pop].cs[cs].current; }

static gc_syn *gc_new_syn(gc_net *net)
{
    if(net->numSyns == net->capSyns) {
        net->capSyns = net->capSyns ? net->capSyns * 2 : 16;
        net->syns = (gc_syn*)realloc(net->syns, net->capSyns * sizeof(gc_syn));
    }
    gc_syn *s = &net->syns[net->numSyns++];
    memset(s, 0, sizeof(*s));
    return s;
}

/* ind / rowLength / d are borrowed (never written); g is copied because STDP writes it */
int gc_add_syn_sparse(gc_net *net, int src, int trg, int psm, int wum, uint32_t rowStride,
                      const uint32_t *rowLength, const uint32_t *ind, const float *g, const uint8_t *d,
                      int copyG)
{
    gc_syn *s = gc_new_syn(net);
    s->matrix = GC_SPARSE; s->wum = wum; s->src = src; s->trg = trg; s->psm = psm;
    s->rowStride = rowStride; s->rowLength = rowLength; s->ind = ind; s->d = d;
    s->g = copyG ? (float*)gc_dup(g, (size_t)net->pops[src].n * rowStride * sizeof(float)) : (float*)g;
    return net->numSyns - 1;
}

/* StaticGraded (weightUpdateModels.h:308-319) on a SPARSE projection added with wum = GC_STATIC_GRADED: the source population
 * gets an event queue for the condition V > Epre — one per distinct threshold, as the reference fuses the event queues of
 * projections whose condition and parameters agree (neuronGroup.cc:505-517) */
void gc_set_static_graded(gc_net *net, int syn, float epre, float vslope)
{
    gc_syn *s = &net->syns[syn];
    gc_pop *p = &net->pops[s->src];
    s->epre = epre; s->vslope = vslope;
    for(int e = 0; e < p->numEvents; e++) {
        if(p->events[e].threshold == epre) { s->event = e; return; }
    }
    s->event = p->numEvents;
    p->events[p->numEvents].threshold = epre;
    p->events[p->numEvents].spkEvent = (uint32_t*)calloc(p->n ? p->n : 1, sizeof(uint32_t));
    p->events[p->numEvents].spkCntEvent = 0;
    p->events[p->numEvents].recordSpkEvent = net->numRec ? (uint32_t*)calloc(net->numRec * ((p->n + 31) / 32), sizeof(uint32_t)) : NULL;
    p->numEvents++;
}

/* A SPARSE projection added with wum = GC_STATIC_REVERSE (presynaptic-spike code `addToPre(g);`): the source gets an outPre */
void gc_set_static_reverse(gc_net *net, int syn)
{
    gc_syn *s = &net->syns[syn];
    gc_pop *p = &net->pops[s->src];
    s->preOutput = p->numPreOutput;
    p->outPre[p->numPreOutput++] = (float*)calloc(p->n ? p->n : 1, sizeof(float));
}

/* sT is initialised to -TIME_MAX (= -FLT_MAX) exactly as the reference's generated initialize() does */
static void gc_need_st(gc_pop *p)
{
    if(!p->sT) {
        p->sT = (float*)malloc(p->n * sizeof(float));
        for(uint32_t i = 0; i < p->n; i++) { p->sT[i] = -3.402823466e+38f; }
    }
}

/* built-in additive STDP with nearest-neighbour pairing (weightUpdateModels.h:345-367): no trace variables, spike times of
 * both populations */
void gc_set_stdp_additive(gc_net *net, int syn, float tauPlus, float tauMinus, float aPlus, float aMinus, float wMin, float wMax,
                          uint32_t colStride)
{
    gc_syn *s = &net->syns[syn];
    gc_pop *pre = &net->pops[s->src], *post = &net->pops[s->trg];
    s->tauPlus = tauPlus; s->tauMinus = tauMinus; s->aPlus = aPlus; s->aMinus = aMinus; s->wMin = wMin; s->wMax = wMax; s->colStride = colStride;
    gc_need_st(pre); gc_need_st(post);
    s->colLength = (uint32_t*)calloc(post->n, sizeof(uint32_t));
    s->remap = (uint32_t*)calloc((size_t)post->n * colStride, sizeof(uint32_t));
}

void gc_set_stdp_trace(gc_net *net, int syn, float aPlus, float aMinus, float wMin, float wMax,
                       float tauPlusDecay, float tauMinusDecay, uint32_t colStride)
{
    gc_syn *s = &net->syns[syn];
    gc_pop *pre = &net->pops[s->src], *post = &net->pops[s->trg];
    s->aPlus = aPlus; s->aMinus = aMinus; s->wMin = wMin; s->wMax = wMax; s->colStride = colStride;
    pre->preTrace = (float*)calloc(pre->n, sizeof(float)); pre->preDecay = tauPlusDecay;
    post->postTrace = (float*)calloc(post->n, sizeof(float)); post->postDecay = tauMinusDecay;
    gc_need_st(pre); gc_need_st(post);
    s->colLength = (uint32_t*)calloc(post->n, sizeof(uint32_t));
    s->remap = (uint32_t*)calloc((size_t)post->n * colStride, sizeof(uint32_t));
}

int gc_add_syn_conv2d(gc_net *net, int src, int trg, int psm, const int *conv, const float *kernel)
{
    gc_syn *s = gc_new_syn(net);
    s->matrix = GC_CONV2D; s->wum = GC_STATIC; s->src = src; s->trg = trg; s->psm = psm;
    memcpy(s->conv, conv, 8 * sizeof(int));
    /* derived parameters conv_bw / conv_bh, initToeplitzConnectivitySnippet.h:113-114 */
    s->conv_bw = ((conv[3] + conv[1] - 1) - conv[6]) / 2;
    s->conv_bh = ((conv[2] + conv[0] - 1) - conv[5]) / 2;
    s->g = (float*)kernel;
    return net->numSyns - 1;
}

/* DENSE (g != NULL: individual weights [numPre*numPost]; else the constant) or BITMASK (gp, rowStride = numPost padded to 32) */
int gc_add_syn_dense(gc_net *net, int src, int trg, int psm, const float *g, float constantWeight)
{
    gc_syn *s = gc_new_syn(net);
    s->matrix = GC_DENSE; s->wum = GC_STATIC; s->src = src; s->trg = trg; s->psm = psm;
    s->g = (float*)g; s->constantWeight = constantWeight;
    return net->numSyns - 1;
}

int gc_add_syn_bitmask(gc_net *net, int src, int trg, int psm, const uint32_t *gp, uint32_t rowStride, float constantWeight)
{
    gc_syn *s = gc_new_syn(net);
    s->matrix = GC_BITMASK; s->wum = GC_STATIC; s->src = src; s->trg = trg; s->psm = psm;
    s->gp = gp; s->rowStride = rowStride; s->constantWeight = constantWeight;
    return net->numSyns - 1;
}

/* backend.cc:156-179 — row-major traversal, so each column lists its synapses in ascending idSyn */
void gc_build_remap(gc_net *net, int syn)
{
    gc_syn *s = &net->syns[syn];
    const uint32_t numPre = net->pops[s->src].n, numPost = net->pops[s->trg].n;
    memset(s->colLength, 0, numPost * sizeof(uint32_t));
    for(uint32_t i = 0; i < numPre; i++) {
        for(uint32_t j = 0; j < s->rowLength[i]; j++) {
            const uint32_t rowMajorIndex = (i * s->rowStride) + j;
            const uint32_t postIndex = s->ind[rowMajorIndex];
            const size_t colMajorIndex = ((size_t)postIndex * s->colStride) + s->colLength[postIndex];
            s->colLength[postIndex]++;
            s->remap[colMajorIndex] = rowMajorIndex;
        }
    }
}

/* ------------------------------------------------------------------------------------------ */
void gc_update_synapses(gc_net *net, float t)
{
    /* dendritic delay pointers advance first */
    for(int p = 0; p < net->numPops; p++) {
        for(int m = 0; m < net->pops[p].numPSM; m++) {
            gc_psm *psm = &net->pops[p].psm[m];
            if(psm->maxDenDelay) { psm->denDelayPtr = (psm->denDelayPtr + 1) % psm->maxDenDelay; }
        }
    }
    /* presynaptic updates: true spikes */
    for(int k = 0; k < net->numSyns; k++) {
        gc_syn *s = &net->syns[k];
        const gc_pop *src = &net->pops[s->src];
        gc_pop *trg = &net->pops[s->trg];
        /* axonal delay: slot (spkQuePtr + slots - delaySteps) % slots of the source's ring (backendBase.cc:207-216) */
        const uint32_t *srcSpk = src->spk;
        uint32_t srcSpkCnt = src->spkCnt;
        if(src->numDelaySlots > 1) {
            const uint32_t slot = (src->spkQuePtr + src->numDelaySlots - s->delaySteps) % src->numDelaySlots;
            srcSpk = src->spkRing + (size_t)slot * src->n;
            srcSpkCnt = src->spkCntRing[slot];
        }
        gc_psm *psm = &trg->psm[s->psm];
        if(s->wum == GC_STATIC_GRADED) {
            /* spike-like events (backend.cc:537-540, the same row loop as true spikes with the event code); V_pre is the
             * source's V as it stands now, i.e. after the update — and reset — of the step that emitted the event */
            const gc_event *ev = &src->events[s->event];
            for(uint32_t i = 0; i < ev->spkCntEvent; i++) {
                const uint32_t idPre = ev->spkEvent[i];
                const uint32_t npost = s->rowLength[idPre];
                s->events += npost;
                for(uint32_t j = 0; j < npost; j++) {
                    const uint32_t idSyn = (idPre * s->rowStride) + j;
                    /* The generated C++ reads `outPost[idPost] += fmax(0.0f, g[idSyn] * tanh((V[idPre] - Epre) / Vslope) * DT)` and
                     * includes only <cmath>, which leaves the double versions of tanh and fmax as the only ones in the global
                     * namespace: the argument is an fp32 quotient, everything after it — the product, the maximum and the
                     * addition to outPost — is double arithmetic, rounded to fp32 by the store. */
                    const float x = (src->v0[idPre] - s->epre) / s->vslope;
                    const double release = fmax((double)0.0f, (double)s->g[idSyn] * tanh((double)x) * (double)net->dt);
                    psm->outPost[s->ind[idSyn]] = (float)((double)psm->outPost[s->ind[idSyn]] + release);
                }
            }
            continue;
        }
        if(s->matrix == GC_CONV2D) {
            const int kh = s->conv[0], kw = s->conv[1], iw = s->conv[3], ic = s->conv[4];
            const int oh = s->conv[5], ow = s->conv[6], oc = s->conv[7];
            const uint32_t rowStride = (uint32_t)(kh * kw * oc);
            for(uint32_t j = 0; j < rowStride; j++) {
                const int32_t kernRow = (int32_t)(j / oc) / kw;
                const int32_t kernCol = (int32_t)(j / oc) % kw;
                const int32_t kernOutChan = (int32_t)(j % oc);
                const int32_t flipKernRow = kh - kernRow - 1;
                const int32_t flipKernCol = kw - kernCol - 1;
                for(uint32_t i = 0; i < srcSpkCnt; i++) {
                    const uint32_t ipre = srcSpk[i];
                    const int32_t preRow = (int32_t)(ipre / ic) / iw;
                    const int32_t preCol = (int32_t)(ipre / ic) % iw;
                    const int32_t preChan = (int32_t)(ipre % ic);
                    const int32_t postRow = preRow + kernRow - s->conv_bh;
                    const int32_t postCol = preCol + kernCol - s->conv_bw;
                    if(postRow >= 0 && postCol >= 0 && postRow < oh && postCol < ow) {
                        const int32_t postInd = (postRow * ow * oc) + (postCol * oc) + kernOutChan;
                        const uint32_t kernelInd = (uint32_t)((flipKernRow * kw * ic * oc) + (flipKernCol * ic * oc) + (preChan * oc) + kernOutChan);
                        psm->outPost[postInd] += s->g[kernelInd];
                        s->events++;
                    }
                }
            }
            continue;
        }
        if(s->matrix == GC_DENSE || s->matrix == GC_BITMASK) {
            /* backend.cc:1985-2021: for every spike, every postsynaptic neuron in ascending order */
            for(uint32_t i = 0; i < srcSpkCnt; i++) {
                const uint32_t idPre = srcSpk[i];
                for(uint32_t ipost = 0; ipost < trg->n; ipost++) {
                    if(s->matrix == GC_BITMASK) {
                        const uint64_t gid = ((uint64_t)idPre * s->rowStride) + ipost;
                        if(s->gp[gid / 32] & (0x80000000u >> (gid & 31))) {
                            psm->outPost[ipost] += s->constantWeight;
                            s->events++;
                        }
                    }
                    else {
                        const size_t idSyn = ((size_t)idPre * trg->n) + ipost;
                        psm->outPost[ipost] += s->g ? s->g[idSyn] : s->constantWeight;
                        s->events++;
                    }
                }
            }
            continue;
        }
        for(uint32_t i = 0; i < srcSpkCnt; i++) {
            const uint32_t idPre = srcSpk[i];
            const uint32_t npost = s->rowLength[idPre];
            s->events += npost;
            for(uint32_t j = 0; j < npost; j++) {
                const uint32_t idSyn = (idPre * s->rowStride) + j;
                const uint32_t idPost = s->ind[idSyn];
                if(s->wum == GC_STATIC) {
                    psm->outPost[idPost] += s->g[idSyn];
                }
                else if(s->wum == GC_STATIC_REVERSE) {
                    /* addToPre(x): outPre[idPre] += x (backend.cc:1822) */
                    net->pops[s->src].outPre[s->preOutput][idPre] += s->g[idSyn];
                }
                else if(s->wum == GC_STATIC_DELAY) {
                    psm->denDelay[(size_t)((psm->denDelayPtr + s->d[idSyn]) % psm->maxDenDelay) * trg->n + idPost] += s->g[idSyn];
                }
                else if(s->wum == GC_STDP_ADDITIVE) {
                    /* weightUpdateModels.h:352-359.  The generated code includes <cmath> only and calls exp unqualified, so
                     * the exponential is the double one, rounded once on assignment to the scalar */
                    const float stPost = net->dt + trg->sT[idPost];
                    psm->outPost[idPost] += s->g[idSyn];
                    const float dt = t - stPost;
                    if(dt > 0) {
                        const float timing = (float)exp((double)(-dt / s->tauMinus));
                        const float newWeight = s->g[idSyn] - (s->aMinus * timing);
                        s->g[idSyn] = fmaxf(s->wMin, fminf(s->wMax, newWeight));
                    }
                }
                else {
                    const float stPost = net->dt + trg->sT[idPost];
                    psm->outPost[idPost] += s->g[idSyn];
                    const float dt = t - stPost;
                    if(dt > 0) {
                        const float newWeight = s->g[idSyn] - (s->aMinus * trg->postTrace[idPost]);
                        s->g[idSyn] = fminf(s->wMax, fmaxf(s->wMin, newWeight));
                    }
                }
            }
        }
    }
    /* postsynaptic updates (learnPost) through the column remap */
    for(int k = 0; k < net->numSyns; k++) {
        gc_syn *s = &net->syns[k];
        if(s->wum != GC_STDP_TRACE && s->wum != GC_STDP_ADDITIVE) { continue; }
        const gc_pop *src = &net->pops[s->src];
        const gc_pop *trg = &net->pops[s->trg];
        const uint32_t numSpikes = trg->spkCnt;
        for(uint32_t j = 0; j < numSpikes; j++) {
            const uint32_t spike = trg->spk[j];
            const uint32_t npre = s->colLength[spike];
            for(uint32_t i = 0; i < npre; i++) {
                const size_t colMajorIndex = ((size_t)spike * s->colStride) + i;
                const uint32_t rowMajorIndex = s->remap[colMajorIndex];
                const uint32_t idPre = rowMajorIndex / s->rowStride;
                const float stPre = net->dt + src->sT[idPre];
                const float dt = t - stPre;
                if(dt > 0 && s->wum == GC_STDP_ADDITIVE) {
                    /* weightUpdateModels.h:360-366 */
                    const float timing = (float)exp((double)(-dt / s->tauPlus));
                    const float newWeight = s->g[rowMajorIndex] + (s->aPlus * timing);
                    s->g[rowMajorIndex] = fmaxf(s->wMin, fminf(s->wMax, newWeight));
                }
                else if(dt > 0) {
                    const float newWeight = s->g[rowMajorIndex] + (s->aPlus * src->preTrace[idPre]);
                    s->g[rowMajorIndex] = fminf(s->wMax, fmaxf(s->wMin, newWeight));
                }
            }
        }
    }
}

void gc_update_neurons(gc_net *net, float t, uint32_t recordingTimestep)
{
    const uint64_t step = net->timestep;
    for(int k = 0; k < net->numPops; k++) {
        gc_pop *p = &net->pops[k];
        if(p->numDelaySlots > 1) {
            p->spkQuePtr = (p->spkQuePtr + 1) % p->numDelaySlots;
            p->spk = p->spkRing + (size_t)p->spkQuePtr * p->n;
        }
        p->spkCnt = 0;
        for(int e = 0; e < p->numEvents; e++) { p->events[e].spkCntEvent = 0; }
    }
    for(int k = 0; k < net->numPops; k++) {
        gc_pop *p = &net->pops[k];
        const uint32_t numRecordingWords = (p->n + 31) / 32;
        uint32_t *rec = p->recordSpk ? &p->recordSpk[(size_t)recordingTimestep * numRecordingWords] : NULL;
        if(rec) { memset(rec, 0, numRecordingWords * sizeof(uint32_t)); }
        /* spike-like event recording buffers are cleared the same way (backend.cc:309-318) */
        for(int e = 0; e < p->numEvents; e++) {
            if(p->events[e].recordSpkEvent) { memset(&p->events[e].recordSpkEvent[(size_t)recordingTimestep * numRecordingWords], 0, numRecordingWords * sizeof(uint32_t)); }
        }
        for(uint32_t i = 0; i < p->n; i++) {
            int spiked;
            if(p->model == GC_SSA) {
                uint32_t startSpike = p->startSpike[i];
                if(p->preTrace) { p->preTrace[i] *= p->preDecay; }
                if(p->postTrace) { p->postTrace[i] *= p->postDecay; }
                spiked = (startSpike != p->endSpike[i] && t >= p->spikeTimes[startSpike]);
                if(spiked) {
                    if(p->preTrace) { p->preTrace[i] += 1.0f; }
                    if(p->postTrace) { p->postTrace[i] += 1.0f; }
                    if(rec) { rec[i / 32] |= (1u << (i % 32)); }
                    if(p->sT) { p->sT[i] = t; }
                    p->spk[p->spkCnt++] = i;
                    startSpike++;
                }
                p->startSpike[i] = startSpike;
                continue;
            }
            float Isyn = 0;
            float l0 = p->v0[i], l1 = p->v1[i];
            for(int m = 0; m < p->numPSM; m++) {
                gc_psm *psm = &p->psm[m];
                float linSyn = psm->outPost[i];
                if(psm->maxDenDelay) {
                    float *denDelayFront = &psm->denDelay[((size_t)psm->denDelayPtr * p->n) + i];
                    linSyn += *denDelayFront;
                    *denDelayFront = 0.0f;
                }
                if(psm->kind == GC_EXPCURR) {
                    Isyn += psm->init * linSyn;
                    linSyn *= psm->expDecay;
                }
                else {
                    Isyn += linSyn;
                    linSyn = 0.0f;
                }
                psm->outPost[i] = linSyn;
            }
            /* presynaptic output: after the incoming postsynaptic models, before the current sources (neuronUpdateGroupMerged.cc:585-600) */
            for(int q = 0; q < p->numPreOutput; q++) {
                Isyn += p->outPre[q][i];
                p->outPre[q][i] = 0.0f;
            }
            for(int c = 0; c < p->numCS; c++) {
                gc_cs *cs = &p->cs[c];
                if(cs->kind == GC_CS_POISSON_EXP) {
                    /* the snippet's loop (uniforms in [0, 1) with 24 significant bits, four per generator call) */
                    float prod = 1.0f;
                    uint32_t numSpikes = 0;
                    int done = 0;
                    for(uint32_t call = 0; !done; call++) {
                        uint32_t r[4];
                        gc_philox4x32(cs->indexOffset + i, (uint32_t)step, call, cs->stream, (uint32_t)cs->seed, (uint32_t)(cs->seed >> 32), r);
                        for(int w = 0; w < 4 && !done; w++) {
                            numSpikes++;
                            prod *= (float)(r[w] >> 8) * (1.0f / 16777216.0f);
                            done = !(prod > cs->expMinusLambda);
                        }
                    }
                    cs->current[i] += cs->init * (float)(numSpikes - 1);
                    Isyn += cs->current[i];
                    cs->current[i] *= cs->expDecay;
                }
                else {
                    Isyn += (cs->kind == GC_CS_DC) ? cs->amp : cs->noise[(size_t)(step % cs->noiseSteps) * p->n + i];
                }
            }
            if(p->model == GC_LIF) {
                /* p = {Ioffset, Rmembrane, Vrest, ExpTC, Vthresh, Vreset, TauRefrac} ; l0 = V, l1 = RefracTime */
                if(l1 <= 0.0f) {
                    const float alpha = ((Isyn + p->p[0]) * p->p[1]) + p->p[2];
                    l0 = alpha - (p->p[3] * (alpha - l0));
                }
                else {
                    l1 -= net->dt;
                }
            }
            else {
                /* p = {a, b, c, d}; l0 = V, l1 = U; left-to-right evaluation of the snippet's expressions */
                if(l0 >= 30.0f) {
                    l0 = p->p[2];
                    l1 += p->p[3];
                }
                l0 += 0.5f * (0.04f * l0 * l0 + 5.0f * l0 + 140.0f - l1 + Isyn) * net->dt;
                l0 += 0.5f * (0.04f * l0 * l0 + 5.0f * l0 + 140.0f - l1 + Isyn) * net->dt;
                l1 += p->p[0] * (p->p[1] * l0 - l1) * net->dt;
                if(l0 > 30.0f) { l0 = 30.0f; }
            }
            /* WU pre / post dynamics run every step, before the threshold test */
            if(p->preTrace) { p->preTrace[i] *= p->preDecay; }
            if(p->postTrace) { p->postTrace[i] *= p->postDecay; }
            /* spike-like event conditions: after the sim code, before the threshold test (neuronUpdateGroupMerged.cc:677-683) */
            for(int e = 0; e < p->numEvents; e++) {
                if(l0 > p->events[e].threshold) {
                    p->events[e].spkEvent[p->events[e].spkCntEvent++] = i;
                    /* backend.cc:360-380 */
                    if(p->events[e].recordSpkEvent) { p->events[e].recordSpkEvent[(size_t)recordingTimestep * numRecordingWords + (i / 32)] |= (1u << (i % 32)); }
                }
            }
            spiked = (p->model == GC_LIF) ? (l1 <= 0.0f && l0 >= p->p[4]) : (l0 >= 29.99f);
            if(spiked) {
                if(p->preTrace) { p->preTrace[i] += 1.0f; }
                if(p->postTrace) { p->postTrace[i] += 1.0f; }
                if(rec) { rec[i / 32] |= (1u << (i % 32)); }
                if(p->sT) { p->sT[i] = t; }
                p->spk[p->spkCnt++] = i;
                if(p->model == GC_LIF) { l0 = p->p[5]; l1 = p->p[6]; }
            }
            p->v0[i] = l0; p->v1[i] = l1;
        }
        if(p->numDelaySlots > 1) { p->spkCntRing[p->spkQuePtr] = p->spkCnt; }
    }
}

void gc_step(gc_net *net)
{
    const float t = net->timestep * net->dt;
    gc_update_synapses(net, t);
    gc_update_neurons(net, t, net->numRec ? (uint32_t)(net->timestep % net->numRec) : 0);
    net->timestep++;
}

/* for callers that run the two halves of a step separately */
void gc_advance(gc_net *net) { net->timestep++; }

void gc_run(gc_net *net, uint64_t steps) { for(uint64_t i = 0; i < steps; i++) { gc_step(net); } }

/* ------------------------------------------------------------------------------------------ */
/* accessors                                                                                   */
/* ------------------------------------------------------------------------------------------ */
uint32_t gc_spike_count(const gc_net *net, int pop) { return net->pops[pop].spkCnt; }
const uint32_t *gc_spikes(const gc_net *net, int pop) { return net->pops[pop].spk; }
float *gc_var(gc_net *net, int pop, int which) { return which ? net->pops[pop].v1 : net->pops[pop].v0; }
uint32_t *gc_start_spike(gc_net *net, int pop) { return net->pops[pop].startSpike; }
float *gc_out_post(gc_net *net, int pop, int psm) { return net->pops[pop].psm[psm].outPost; }
float *gc_den_delay(gc_net *net, int pop, int psm) { return net->pops[pop].psm[psm].denDelay; }
uint32_t gc_den_delay_ptr(const gc_net *net, int pop, int psm) { return net->pops[pop].psm[psm].denDelayPtr; }
float *gc_pre_trace(gc_net *net, int pop) { return net->pops[pop].preTrace; }
float *gc_post_trace(gc_net *net, int pop) { return net->pops[pop].postTrace; }
float *gc_spike_time(gc_net *net, int pop) { return net->pops[pop].sT; }
uint32_t *gc_record(gc_net *net, int pop) { return net->pops[pop].recordSpk; }
float *gc_syn_g(gc_net *net, int syn) { return net->syns[syn].g; }
uint32_t *gc_col_length(gc_net *net, int syn) { return net->syns[syn].colLength; }
uint32_t *gc_remap(gc_net *net, int syn) { return net->syns[syn].remap; }
float *gc_out_pre(gc_net *net, int syn) { return net->pops[net->syns[syn].src].outPre[net->syns[syn].preOutput]; }
uint32_t gc_event_count(const gc_net *net, int pop, int event) { return net->pops[pop].events[event].spkCntEvent; }
const uint32_t *gc_events(const gc_net *net, int pop, int event) { return net->pops[pop].events[event].spkEvent; }
uint32_t *gc_event_record(gc_net *net, int pop, int event) { return net->pops[pop].events[event].recordSpkEvent; }
int gc_syn_event_queue(const gc_net *net, int syn) { return net->syns[syn].event; }
uint64_t gc_syn_events(const gc_net *net, int syn) { return net->syns[syn].events; }
uint64_t gc_timestep(const gc_net *net) { return net->timestep; }

void gc_destroy(gc_net *net)
{
    /* arrays are small relative to process lifetime in tests; free the owned ones */
    for(int k = 0; k < net->numPops; k++) {
        gc_pop *p = &net->pops[k];
        free(p->v0); free(p->v1); free(p->startSpike); free((void*)p->endSpike);
        for(int m = 0; m < p->numPSM; m++) { free(p->psm[m].outPost); free(p->psm[m].denDelay); }
        free(p->preTrace); free(p->postTrace); free(p->sT); free(p->recordSpk);
        for(int c = 0; c < p->numCS; c++) { free(p->cs[c].current); }
        if(p->spkRing) { free(p->spkRing); free(p->spkCntRing); } else { free(p->spk); }
        for(int e = 0; e < p->numEvents; e++) { free(p->events[e].spkEvent); free(p->events[e].recordSpkEvent); }
        for(int q = 0; q < p->numPreOutput; q++) { free(p->outPre[q]); }
    }
    for(int k = 0; k < net->numSyns; k++) { free(net->syns[k].colLength); free(net->syns[k].remap); }
    free(net->pops); free(net->syns); free(net);
}
