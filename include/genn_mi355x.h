/*
 * genn_mi355x.h — C ABI of the MI355X (gfx950) device layer for GeNN's per-timestep hot path.
 *
 * Everything a generated runner needs to step a spiking network on one MI355X without
 * containing any device code itself: the runner is plain host C++ that fills merged-group
 * descriptors (the counterpart of the reference's pushMerged<Name>Group<i>ToDevice calls) and
 * calls the entry points below.  Signatures use plain pointers and sizes only.
 *
 * Every function returns 0 on success or a negative GENNMI_E* code; gennmi_last_error()
 * returns a description of the last failure on the calling thread.  The reference signals
 * the same conditions by throwing std::runtime_error from CHECK_RUNTIME_ERRORS
 * (src/genn/backends/hip/backend.cc:696-701); a C++ runner turns a non-zero return into that.
 *
 * All device pointers are addresses returned by gennmi_malloc (or any hipMalloc'd memory of
 * the same process).  Memory is owned by the caller — the reference's Runtime owns arrays
 * through backend Array objects and the runner only receives pointers
 * (src/genn/genn/runtime/runtime.cc:147-402, include/genn/genn/runtime/runtime.h:573-669).
 */
#ifndef GENN_MI355X_H
#define GENN_MI355X_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define GENNMI_OK            0
#define GENNMI_EHIP         -1   /* a HIP runtime call failed */
#define GENNMI_EINVAL       -2   /* descriptor inconsistent with what the kernels assume */
#define GENNMI_EUNSUPPORTED -3   /* feature outside the supported model set */
#define GENNMI_ESTATE       -4   /* call order violated (e.g. step before finalise) */
#define GENNMI_EDEVICE      -5   /* a kernel reported an internal failure (bounded wait expired) */

#define GENNMI_MAX_PSM 8         /* fused postsynaptic models per neuron group */
#define GENNMI_MAX_CS  4         /* current sources per neuron group */
#define GENNMI_MAX_EXTRA_SPK 3   /* spike arrays per neuron group beyond the first */

/* neuron models: include/genn/genn/neuronModels.h:220-257 (LIF), :163-186 (Izhikevich), :274-286 (SpikeSourceArray) */
enum { GENNMI_NEURON_LIF = 0, GENNMI_NEURON_IZHIKEVICH = 1, GENNMI_NEURON_SPIKE_SOURCE_ARRAY = 2 };
/* postsynaptic models: include/genn/genn/postsynapticModels.h:91-106 (ExpCurr), DeltaCurr */
enum { GENNMI_PSM_EXPCURR = 0, GENNMI_PSM_DELTACURR = 1 };
/* current sources: include/genn/genn/currentSourceModels.h:70-77 (DC); ARRAY injects noise[step*numNeurons+id] */
enum { GENNMI_CS_DC = 0, GENNMI_CS_ARRAY = 1, GENNMI_CS_POISSON_EXP = 2 };
/* weight update models: include/genn/genn/weightUpdateModels.h:236-244, :279-287; trace STDP pygenn/genn_model.py:1448-1476 */
enum { GENNMI_WUM_STATIC_PULSE = 0, GENNMI_WUM_STATIC_PULSE_DENDRITIC_DELAY = 1, GENNMI_WUM_STDP_TRACE = 2,
       GENNMI_WUM_STATIC_PULSE_CONSTANT_WEIGHT = 3, /* weightUpdateModels.h:202-213: one weight for the whole projection */
       /* weightUpdateModels.h:308-319: no spike code; while the presynaptic V exceeds Epre the neuron emits a spike-like
        * event every step, and each event adds fmax(0, g * tanh((V_pre - Epre) / Vslope) * dt) per synapse */
       GENNMI_WUM_STATIC_GRADED = 4,
       /* presynaptic-spike code `addToPre(g);` (the static_pulse_reverse model of tests/features/test_event_propagation.py:584-590):
        * every synapse of a spiking neuron's row adds its weight to that neuron's own outPre (SPARSE only) */
       GENNMI_WUM_STATIC_PULSE_REVERSE = 5,
       /* the built-in additive STDP with nearest-neighbour pairing (weightUpdateModels.h:345-367): a presynaptic spike
        * delivers g, then g = clamp(g - Aminus * exp(-(t - st_post) / tauMinus)); a postsynaptic spike applies
        * g = clamp(g + Aplus * exp(-(t - st_pre) / tauPlus)) down its column.  The exponential is the double one, rounded
        * once, as in the code the reference generates for its CPU backend.  No trace arrays. */
       GENNMI_WUM_STDP = 6 };
/* connectivity: ragged SPARSE (runtime.cc:360-402) or TOEPLITZ Conv2D (initToeplitzConnectivitySnippet.h:105-150) */
enum { GENNMI_MATRIX_SPARSE = 0, GENNMI_MATRIX_TOEPLITZ_CONV2D = 1,
       /* DENSE: g[numSrc*numTrg], idSyn = idPre*numTrg + idPost; BITMASK: one bit per pair, most significant bit first,
        * gid = idPre*rowStride + idPost with rowStride = numTrg padded to 32 (single_threaded_cpu/backend.cc:1393-1404,
        * 1985-2021; runtime.cc:340-357) */
       GENNMI_MATRIX_DENSE = 2, GENNMI_MATRIX_BITMASK = 3,
       /* PROCEDURAL (synapseMatrixType.h:60-66; presynapticUpdateStrategySIMT.cc:391-560): nothing is stored, the row of a
        * spiking neuron — and its weights — are regenerated from the initialisation snippets' generator when needed */
       GENNMI_MATRIX_PROCEDURAL = 4 };
enum { GENNMI_CONNECT_FIXED_PROBABILITY = 0, GENNMI_CONNECT_FIXED_PROBABILITY_NO_AUTAPSE = 1, GENNMI_CONNECT_FIXED_NUMBER_POST = 2 };
/* presynaptic strategies: presynapticUpdateStrategySIMT.cc:57-162 (PreSpan), :167-389 (PostSpan) */
enum { GENNMI_SPAN_AUTO = 0, GENNMI_SPAN_POST = 1, GENNMI_SPAN_PRE = 2 };

/* ---------------------------------------------------------------------------------------------
 * Thin device layer.  Replaces the hip* calls the reference emits inline into generated code and
 * its Array class (src/genn/backends/hip/backend.cc:61-236: allocate/free/push/pull/memset).
 * ------------------------------------------------------------------------------------------- */
int gennmi_init(int device);                                   /* hip/backend.cc:290-322 (device select) */
const char *gennmi_last_error(void);
int gennmi_device_name(char *buf, size_t len);
int gennmi_malloc(void **devPtr, size_t bytes);                 /* Array::allocate  hip/backend.cc:86-108 */
/* Pinned, zero-filled host memory for an array's host side (hipHostMalloc in Array::allocate, hip/backend.cc:90-97).  With
 * `zeroCopy` (VarLocation::HOST_DEVICE_ZERO_COPY) the memory is mapped into the device's address space and *devPtr receives
 * the address kernels use (hipHostGetDevicePointer, :101-103): such an array has no device buffer of its own and needs no
 * copies.  Without it devPtr may be NULL.  gennmi_host_free releases the memory. */
int gennmi_host_malloc(void **hostPtr, size_t bytes, int zeroCopy, void **devPtr);
int gennmi_host_free(void *hostPtr);
int gennmi_free(void *devPtr);                                  /* Array::free      hip/backend.cc:110-128 */
int gennmi_memcpy_to_device(void *dev, const void *host, size_t bytes);    /* pushToDevice / pushSlice1DToDevice   :130-176 */
int gennmi_memcpy_from_device(void *host, const void *dev, size_t bytes);  /* pullFromDevice / pullSlice1DFromDevice :142-198 */
int gennmi_memset(void *dev, int value, size_t bytes);          /* memsetDeviceObject :200-204 */
int gennmi_fill_f32(float *dev, float value, size_t count);     /* e.g. sT = -TIME_MAX (initGroupMerged.cc neuron init) */
/* Device-to-device copy of `count` floats by a plain kernel (one 16-byte load and store per lane).  No counterpart
 * in the reference, whose arrays are only copied between host and device; it exists for host code that
 * snapshots state on the device, and as the traffic yardstick hardware counters are scaled by (a launch moves
 * exactly 8*count bytes). */
int gennmi_copy_f32(float *dst, const float *src, size_t count);
int gennmi_synchronize(void);
/* No counterpart in the reference.  Arrays handed to a runner stay the caller's: it may write them by its own means (a
 * hipMemcpy of its own, a kernel of its own) instead of through the calls above.  The library keeps copies derived from
 * some of them — the resident plan's segment tables and packed synapse records (weights, targets, delays), the tile path's
 * segment boundaries and records, the zero-delay lists of the single-launch step, column views, spike bitmaps — and
 * refreshes them before the next step when it knows the array was written; the calls above tell it, this call is for
 * writes it cannot see.  Cheap; naming a range that feeds no copy does nothing. */
int gennmi_note_device_write(const void *dev, size_t bytes);
/* No counterpart in the reference.  For callers that launch kernels of their own between steps (the custom updates the
 * GeNN backend generates beside the library's step kernels): gennmi_flush runs whatever gennmi_step() calls are still
 * queued (see gennmi_runner_set_step_queue), so that work launched next on the null stream sees their results — the
 * runners' streams are blocking streams, ordered against the null stream in both directions.  gennmi_note_mirror_write is
 * gennmi_note_device_write for the whole device buffer registered behind the host buffer `host` points into. */
int gennmi_flush(void);
int gennmi_note_mirror_write(const void *host);
/* Host mirrors.  GeNN's Runtime serialises HOST pointers into merged-group structs for backends that report
 * isArrayDeviceObjectRequired() == false (runtime.cc:700-720, 1027-1044) — which lets the generated initialize() /
 * initializeSparse() run the reference's own host-side initialisation code on those pointers.  An Array
 * (BackendBase::createArray, hip/backend.cc:61-236) registers its host buffer with the device buffer behind it;
 * generated code translates a host pointer (anywhere inside a registered buffer) to the device address, and
 * gennmi_push_mirrors() uploads every registered buffer (end of initialize() / initializeSparse()). */
int gennmi_register_mirror(const void *host, void *dev, size_t bytes);
int gennmi_unregister_mirror(const void *host);
int gennmi_mirror_device_pointer(const void *host, void **dev);   /* NULL host -> NULL device, no error */
int gennmi_push_mirrors(void);
/* Arrays a device generator fills, and arrays without a host copy (VarLocation::DEVICE, varLocation.h:20-27; the reference's
 * Array allocates no host memory for them, hip/backend.cc:75-90).  No counterparts in the reference, whose GPU backends
 * initialise in kernels and never upload afterwards.
 *  - gennmi_mirrors_begin_initialisation(): first statement of initialize(): forgets which buffers were device-initialised.
 *  - gennmi_mirror_device_initialised(host): a gennmi_init_* call has just filled the device buffer behind `host`:
 *    gennmi_push_mirrors() leaves it alone from now on, and the host copy counts as stale.
 *  - gennmi_mirror_ensure_host(host): called before host code READS such a buffer (per-row initialisation code that walks
 *    rowLength / ind): copies it back if it is stale.
 *  - gennmi_register_device_array: gennmi_register_mirror for an array the model keeps on the device only: `host` is
 *    page-aligned, lazily committed address space (mmap with MAP_NORESERVE) that serves as the array's key in merged
 *    groups and as staging for host-side initialisation code; gennmi_push_mirrors() returns its pages to the system
 *    after uploading, so that such an array holds no host memory once initialisation is over. */
int gennmi_register_device_array(const void *host, void *dev, size_t bytes);
int gennmi_mirrors_begin_initialisation(void);
int gennmi_mirror_device_initialised(const void *host);
int gennmi_mirror_ensure_host(const void *host);
int gennmi_free_device_memory_bytes(size_t *bytes);
/* Named ranges for profilers around stepTime / updateSynapses / updateNeurons (BackendBase::genPushProfilerRange /
 * genPopProfilerRange, backendBase.h:345-349; nvtxRangePushA / nvtxRangePop in cuda/backend.cc:741-752): roctxRangePushA /
 * roctxRangePop of libroctx64, looked up when first called; without that library the calls do nothing.  Both return
 * GENNMI_OK. */
int gennmi_profiler_range_push(const char *name);
int gennmi_profiler_range_pop(void);             /* genReturnFreeDeviceMemoryBytes, backendCUDAHIP.cc */
/* sizeof() of the five descriptor structs below, in declaration order (psm, cs, neuron update, presynaptic
 * update, postsynaptic update), so that a binding in another language can verify its struct layout.  Needs
 * no device.  The reference gets the same guarantee from generating both sides of every push call from one
 * field list (groupMerged.h:214-227). */
int gennmi_abi_struct_sizes(size_t sizes[5]);

/* ---------------------------------------------------------------------------------------------
 * Merged-group descriptors.  Field names follow the reference's merged structs
 * (src/genn/genn/code_generator/backendBase.cc:104-380); one descriptor = one group of one
 * merged group, i.e. one pushMerged<Name>Group<i>ToDevice(idx, ...) call.
 * Per-neuron arrays hold batchSize*numNeurons elements, batch-major.
 * ------------------------------------------------------------------------------------------- */
typedef struct gennmi_psm_t {             /* one fused postsynaptic model ("InSyn" child, neuronUpdateGroupMerged.cc:66-137) */
    float *outPost;                       /* [batch*numNeurons] */
    float *denDelay;                      /* [batch*maxDenDelay*numNeurons] slot-major, or NULL */
    uint32_t *denDelayPtr;                /* [1] device-resident head pointer, or NULL */
    float init, expDecay;                 /* ExpCurr derived parameters, already rounded to fp32 */
    uint32_t kind;                        /* GENNMI_PSM_* */
    uint32_t maxDenDelay;                 /* 0 = no dendritic delay */
} gennmi_psm_t;

typedef struct gennmi_cs_t {              /* one current source child (neuronUpdateGroupMerged.cc:20-55) */
    const float *array;                   /* GENNMI_CS_ARRAY: [numSteps*numNeurons]; row (step % arraySteps) is injected */
    float amp;                            /* GENNMI_CS_DC */
    uint32_t kind;
    uint32_t arraySteps;
    /* GENNMI_CS_POISSON_EXP (currentSourceModels.h:100-129): numSpikes ~ Poisson(rate*dt) by the snippet's product-of-uniforms
     * loop, current += Init*numSpikes, injected, then current *= ExpDecay.  The uniforms of neuron i (batch-major index) in
     * step k are the words of Philox4x32-10(counter = (i, k, call, stream), key = seed), call = 0, 1, ... as the loop needs them. */
    uint32_t stream;
    float *current;                       /* state variable [batch*numNeurons] */
    float init, expDecay, expMinusLambda; /* the snippet's derived parameters, rounded to fp32 */
    uint32_t pad_;
    uint64_t seed;
} gennmi_cs_t;

/* Spike-like events ("SynSpikeEvent" children, neuronUpdateGroupMerged.cc:189-330): after the neuron's sim code and
 * before its threshold test, a neuron whose V exceeds `threshold` is appended to this queue (ascending neuron index, like
 * true spikes; backend.cc genEmitEvent).  The queue is rewritten every step.  Projections whose weight update model has
 * an event threshold read it as their srcSpk / srcSpkCnt. */
#define GENNMI_MAX_SPK_EVENT 2
#define GENNMI_MAX_PRE_OUTPUT 2
typedef struct gennmi_spike_event_t {
    uint32_t *spkCntEvent;                /* [batch] */
    uint32_t *spkEvent;                   /* [batch*numNeurons] */
    uint32_t *recordSpkEvent;             /* [numRecordingTimesteps*batch*ceil(numNeurons/32)] or NULL: the events of every step as a
                                           * bitfield, laid out like recordSpk (runtime.cc:307-311) */
    float threshold;                      /* StaticGraded: Epre */
    uint32_t pad_;
} gennmi_spike_event_t;

typedef struct gennmi_neuron_update_group_t {      /* MergedNeuronUpdateGroup<i> */
    uint32_t model;                       /* GENNMI_NEURON_* */
    uint32_t numNeurons;
    float *var0, *var1;                   /* LIF: V, RefracTime.  Izhikevich: V, U */
    uint32_t *startSpike;                 /* SpikeSourceArray state [batch*numNeurons] */
    const uint32_t *endSpike;             /* [batch*numNeurons] */
    const float *spikeTimes;              /* shared across batches */
    /* LIF: Ioffset, Rmembrane, Vrest, ExpTC, Vthresh, Vreset, TauRefrac.  Izhikevich: a, b, c, d. */
    float params[8];
    uint32_t numPSM, numCS;
    gennmi_psm_t psm[GENNMI_MAX_PSM];
    gennmi_cs_t cs[GENNMI_MAX_CS];
    float *preTrace, *postTrace;          /* fused WU pre / post variables (OutSynWUMPre / InSynWUMPost children), or NULL */
    float preDecay, postDecay;
    float *sT;                            /* spike times [batch*numNeurons] or NULL */
    uint32_t *spkCnt;                     /* [batch * max(1, numDelaySlots)] */
    uint32_t *spk;                        /* [batch * max(1, numDelaySlots) * numNeurons], ascending neuron index within a step */
    uint32_t *recordSpk;                  /* [numRecordingTimesteps*batch*ceil(numNeurons/32)] or NULL (runtime.cc:169) */
    /* further spike arrays that receive the same queue: the reference keeps one srcSpk per fused outgoing spike
     * owner and one trgSpk per incoming projection with learnPost (runtime.cc:267-278, "SynSpike" children) */
    uint32_t numExtraSpk;
    /* Axonal delay (backendBase.cc:128-162, neuronUpdateGroupMerged.cc:947-953): with numDelaySlots > 1 the queue is a ring
     * of slots, slot-major within a batch; the step that follows k completed steps writes slot (k + 1) % numDelaySlots
     * (the reference's spkQuePtr after its increment at the start of updateNeurons).  0 or 1: no delay. */
    uint32_t numDelaySlots;
    uint32_t *extraSpkCnt[GENNMI_MAX_EXTRA_SPK];
    uint32_t *extraSpk[GENNMI_MAX_EXTRA_SPK];
    uint32_t numSpkEvent;                 /* LIF and Izhikevich groups without delay slots only */
    /* Presynaptic output ("OutSynPreOutput" children, neuronUpdateGroupMerged.cc:148-165): after the postsynaptic models and
     * before the current sources, Isyn += outPre[id]; outPre[id] = 0 for each outgoing projection whose code calls addToPre */
    uint32_t numPreOutput;
    gennmi_spike_event_t spkEvent[GENNMI_MAX_SPK_EVENT];
    float *outPre[GENNMI_MAX_PRE_OUTPUT]; /* [batch*numNeurons] each */
} gennmi_neuron_update_group_t;

/* What gennmi_init_sparse_* and gennmi_init_var would have stored for a projection, for GENNMI_MATRIX_PROCEDURAL: the row
 * of presynaptic neuron r is row r of that connectivity call (same seed and stream), truncated to rowStride entries, and
 * the weight of its k-th synapse is element r*rowStride + k of that gennmi_init_var call. */
typedef struct gennmi_procedural_t {
    uint64_t seed;
    uint32_t connectivity;                /* GENNMI_CONNECT_* */
    uint32_t connectivityStream;
    double prob;                          /* FixedProbability[NoAutapse] */
    uint32_t num;                         /* FixedNumberPostWithReplacement */
    uint32_t weightSnippet;               /* GENNMI_INIT_CONSTANT .. GENNMI_INIT_EXPONENTIAL */
    uint32_t weightStream, pad_;
    double weightParams[4];
} gennmi_procedural_t;

typedef struct gennmi_presynaptic_update_group_t { /* MergedPresynapticUpdateGroup<i> */
    uint32_t matrix;                      /* GENNMI_MATRIX_* */
    uint32_t wum;                         /* GENNMI_WUM_* */
    uint32_t span;                        /* GENNMI_SPAN_* (parallelism hint, synapseGroup.h:42-47) */
    uint32_t numThreadsPerSpike;          /* PreSpan only (synapseGroup.h:135) */
    uint32_t numSrcNeurons, numTrgNeurons;
    uint32_t rowStride;
    uint32_t maxDenDelay;
    const uint32_t *rowLength;            /* [numSrcNeurons] */
    const uint32_t *ind;                  /* [numSrcNeurons*rowStride] */
    float *g;                             /* [numSrcNeurons*rowStride], or Toeplitz kernel [kh*kw*ic*oc] */
    const uint8_t *d;                     /* [numSrcNeurons*rowStride] dendritic delay in timesteps */
    float *outPost;                       /* fused PSM target of this group */
    float *denDelay;
    uint32_t *denDelayPtr;
    const uint32_t *srcSpkCnt, *srcSpk;
    const float *trgST;                   /* STDP: postsynaptic spike times */
    const float *postTrace;
    float aMinus, wMin, wMax;
    int32_t conv[8];                      /* conv_kh, conv_kw, conv_ih, conv_iw, conv_ic, conv_oh, conv_ow, conv_oc */
    const uint32_t *gp;                   /* BITMASK: [ceil(numSrcNeurons*rowStride / 32)] connectivity words */
    float constantWeight;                 /* GENNMI_WUM_STATIC_PULSE_CONSTANT_WEIGHT: the parameter g (DENSE and BITMASK) */
    /* Axonal delay: the projection reads the source's slot (spkQuePtr + numSrcDelaySlots - axonalDelaySteps) %
     * numSrcDelaySlots (backendBase.cc:207-216), i.e. the spikes emitted axonalDelaySteps + 1 steps before the step that
     * delivers them.  numSrcDelaySlots must equal the source group's numDelaySlots (0 or 1: no ring). */
    uint32_t axonalDelaySteps;
    uint32_t numSrcDelaySlots;
    float tauMinus;                       /* GENNMI_WUM_STDP */
    gennmi_procedural_t procedural;       /* GENNMI_MATRIX_PROCEDURAL only (rowStride = the stride the stored matrix would have) */
    /* GENNMI_WUM_STATIC_GRADED (SPARSE only): srcSpk / srcSpkCnt are the source's event queue for threshold Epre; V_pre is
     * read when the event is delivered, i.e. after the update (and reset) that emitted it */
    const float *srcV;                    /* [batch*numSrcNeurons] the source population's V */
    float gradedEpre, gradedVslope;
    float *outPre;                        /* GENNMI_WUM_STATIC_PULSE_REVERSE: [batch*numSrcNeurons], the source's presynaptic output */
} gennmi_presynaptic_update_group_t;

typedef struct gennmi_postsynaptic_update_group_t { /* MergedPostsynapticUpdateGroup<i> */
    uint32_t numSrcNeurons, numTrgNeurons;
    uint32_t rowStride, colStride;
    const uint32_t *colLength;            /* [numTrgNeurons] */
    const uint32_t *remap;                /* [numTrgNeurons*colStride] */
    float *g;
    const uint32_t *trgSpkCnt, *trgSpk;
    const float *srcST, *preTrace;
    float aPlus, wMin, wMax;
    float tauPlus;                        /* > 0: the built-in additive rule (GENNMI_WUM_STDP), preTrace unused; 0: trace STDP */
    /* row view of the same matrix (optional, both or neither): lets a step in which a large share of the target
     * population fired walk the rows once, coalesced, instead of one gather per (spike, column entry) */
    const uint32_t *rowLength;            /* [numSrcNeurons] */
    const uint32_t *ind;                  /* [numSrcNeurons*rowStride] */
} gennmi_postsynaptic_update_group_t;

/* ---------------------------------------------------------------------------------------------
 * Runner: the device-side half of one generated librunner.so.
 * ------------------------------------------------------------------------------------------- */
typedef struct gennmi_runner gennmi_runner;

/* allocateMem()  generateRunner.cc:241-252.  dt is the fp32 time-precision literal of the model's DT. */
int gennmi_runner_create(gennmi_runner **runner, float dt, uint32_t batchSize);
/* freeMem()  generateRunner.cc:256-265 */
int gennmi_runner_destroy(gennmi_runner *runner);

/* pushMergedNeuronUpdateGroup<i>ToDevice(idx, fields...)  backendCUDAHIP.h:206-238, runtime.h:573-669.
 * Groups are appended; *idx receives the position.  Pushing is only legal before finalise. */
int gennmi_push_neuron_update_group(gennmi_runner *runner, const gennmi_neuron_update_group_t *group, uint32_t *idx);
int gennmi_push_presynaptic_update_group(gennmi_runner *runner, const gennmi_presynaptic_update_group_t *group, uint32_t *idx);
int gennmi_push_postsynaptic_update_group(gennmi_runner *runner, const gennmi_postsynaptic_update_group_t *group, uint32_t *idx);

/* Ordered accumulation, a validation mode (no counterpart in the reference's GPU backends, whose sums are in atomic
 * order like this library's default): every SPARSE projection with StaticPulse, StaticPulseDendriticDelay or an STDP rule is
 * gathered per postsynaptic neuron through a column view of its matrix, spikes in queue order and synapses in ascending
 * index, projections one after another in push order — the order of the SingleThreadedCPU backend's loops
 * (src/genn/backends/single_threaded_cpu/backend.cc:1884-1929) — so outPost, the dendritic-delay rings and everything
 * downstream are bit-identical to that backend's, not merely within reassociation error.  No atomics, no tile,
 * single-launch or resident plan; it reads every column every step, so it is slow.  Call before gennmi_runner_finalise;
 * GENNMI_ORDERED=1 in the environment selects it for every runner.  Bit 3 of info[0] (gennmi_runner_get_info) reports it. */
int gennmi_runner_set_ordered(gennmi_runner *runner, int enabled);

/* Validates descriptors against the kernels' assumptions, uploads the descriptor tables, fixes
 * the launch geometry.  Corresponds to the end of Runtime::allocate (runtime.cc:497-661). */
int gennmi_runner_finalise(gennmi_runner *runner);

/* initializeSparse(): builds colLength / remap for one SPARSE matrix with the reference's CPU
 * ordering (ascending idSyn within a column; single_threaded_cpu/backend.cc:156-179), replacing
 * the order-nondeterministic atomic build of backendSIMT.cc:1977-1991. */
int gennmi_build_remap(uint32_t numSrcNeurons, uint32_t numTrgNeurons, uint32_t rowStride, uint32_t colStride,
                       const uint32_t *rowLength, const uint32_t *ind, uint32_t *colLength, uint32_t *remap);
/* ---------------------------------------------------------------------------------------------
 * On-device initialisation: what the reference's GPU backends run in initializeKernel /
 * initializeSparseKernel (src/genn/genn/code_generator/backendSIMT.cc:1482-1779) for its built-in snippets.
 * Every draw is Philox4x32-10 of (seed, stream, element or row, draw number), so results do not depend on
 * the launch geometry; like the reference's GPU backends (hiprand Philox, src/genn/backends/hip/backend.cc:32-50)
 * the values differ from the CPU backend's std::mt19937 draws and agree with them in distribution only
 * (the reference tests that much: tests/features/test_connect_init.py, test_rng.py).  All launches go to the
 * null stream; the connectivity calls return after the kernel has finished.
 * ------------------------------------------------------------------------------------------- */
/* value snippets, include/genn/genn/initVarSnippet.h: Constant :87-95 {constant}; Uniform :120-130 {min, max};
 * Normal :140-148 {mean, sd}; NormalClipped :161-175 {mean, sd, min, max}; NormalClippedDelay :190-209 {mean, sd, min, max
 * already divided by dt, as the snippet's derived parameters}; Exponential :218-226 {lambda}; Gamma :236-244 {a, b};
 * Binomial :254-262 {n, p} */
enum { GENNMI_INIT_CONSTANT = 0, GENNMI_INIT_UNIFORM = 1, GENNMI_INIT_NORMAL = 2, GENNMI_INIT_NORMAL_CLIPPED = 3,
       GENNMI_INIT_NORMAL_CLIPPED_DELAY = 4, GENNMI_INIT_EXPONENTIAL = 5, GENNMI_INIT_GAMMA = 6, GENNMI_INIT_BINOMIAL = 7 };
enum { GENNMI_TYPE_F32 = 0, GENNMI_TYPE_U32 = 1, GENNMI_TYPE_I32 = 2, GENNMI_TYPE_U16 = 3, GENNMI_TYPE_U8 = 4 };
/* genVariableInit / genSparseSynapseVariableRowInit (backendBase.h:246-251): fills `count` elements of a 16-byte aligned
 * device array; values are computed in fp32 and converted to the element type.  Per-synapse variables of a SPARSE
 * matrix are filled over the whole numPre*rowStride range, padding included (padding is never read). */
int gennmi_init_var(void *dev, uint32_t elementType, size_t count, uint32_t snippet, const double params[4], uint64_t seed, uint32_t stream);
/* FixedProbability (initSparseConnectivitySnippet.h:170-187) and FixedProbabilityNoAutapse (:208-230): rows ascending.
 * Rows that draw more than rowStride entries are truncated, counted in *overflowRows (may be NULL) and make the call
 * return GENNMI_EINVAL; the reference sizes rowStride so that this has probability 1e-4 per matrix (:135-142). */
int gennmi_init_sparse_fixed_probability(uint32_t numPre, uint32_t numPost, uint32_t rowStride, double prob, int noAutapse,
                                         uint64_t seed, uint32_t stream, uint32_t *rowLength, uint32_t *ind, uint32_t *overflowRows);
/* FixedNumberPostWithReplacement (:242-276): `num` ascending targets per row.  With rowLengthIn != NULL (device array of
 * numPre counts) row r draws rowLengthIn[r] targets instead: FixedNumberTotalWithReplacement (:292-370), whose row lengths
 * the reference too draws on the host (its host init code) and hands to the device.  rowLengthIn may alias rowLength. */
int gennmi_init_sparse_fixed_number_post(uint32_t numPre, uint32_t numPost, uint32_t rowStride, uint32_t num, const uint32_t *rowLengthIn,
                                         uint64_t seed, uint32_t stream, uint32_t *rowLength, uint32_t *ind, uint32_t *overflowRows);
/* FixedNumberPreWithReplacement (:380-410): every postsynaptic neuron draws `num` sources with replacement (idPre =
 * gennrand() % numPre, the snippet's own arithmetic); a column therefore holds exactly `num` entries, multiplicities counted.
 * Rows are appended to in arbitrary order and then sorted, so they come out ascending like every other generator's;
 * rowStride <= 16384.  Row lengths are Binomial(num * numPost, 1 / numPre): the reference sizes rowStride for the 0.9999
 * quantile (:391-400); rows beyond it are truncated and counted as for the other generators. */
int gennmi_init_sparse_fixed_number_pre(uint32_t numPre, uint32_t numPost, uint32_t rowStride, uint32_t num,
                                        uint64_t seed, uint32_t stream, uint32_t *rowLength, uint32_t *ind, uint32_t *overflowRows);
/* Conv2D as SPARSE connectivity (:438-497): conv = {kh, kw, sh, sw, padh, padw, ih, iw, ic, oh, ow, oc}, the snippet's row
 * build code per presynaptic neuron, targets ascending; rowStride >= ceil(kh / sh) * ceil(kw / sw) * oc (:485-491).  With
 * `kernel` (device array [kh][kw][ic][oc]) and `g`, every synapse's weight is the kernel entry named by its (kernel row,
 * kernel column, input channel, output channel): InitVarSnippet::Kernel (initVarSnippet.h:100-108).  Both NULL: connectivity only. */
int gennmi_init_sparse_conv2d(const int32_t conv[12], uint32_t rowStride, uint32_t *rowLength, uint32_t *ind, const float *kernel, float *g,
                              uint32_t *overflowRows);
/* OneToOne (:107-118) */
int gennmi_init_sparse_one_to_one(uint32_t numPre, uint32_t numPost, uint32_t rowStride, uint32_t *rowLength, uint32_t *ind);
/* The generator itself, for known-answer tests: one Philox4x32-10 block on the host, and the raw words of a stream
 * on the device (word i = output i%4 of counter (i/4, 0, 0, stream) under key = seed). */
int gennmi_philox4x32(const uint32_t counter[4], const uint32_t key[2], uint32_t out[4]);
int gennmi_init_random_words(uint32_t *dev, size_t count, uint64_t seed, uint32_t stream);

/* Longest column of a SPARSE matrix (what SynapseGroup::getMaxSourceConnections must cover). */
int gennmi_max_col_length(uint32_t numSrcNeurons, uint32_t numTrgNeurons, uint32_t rowStride,
                          const uint32_t *rowLength, const uint32_t *ind, uint32_t *maxColLength);

/* gennmi_max_col_length for callers that cannot allocate device memory (tight serving loops, harnesses that forbid
 * hipMalloc).  It has no counterpart in the reference.  The per-column counters live in an array
 * that is part of the library's device image (GENNMI_STATIC_MAX_TARGETS counters = 4 MiB on every GPU the library runs
 * on, held until the process ends), so the call allocates and frees nothing; numTrgNeurons above that limit is rejected
 * with GENNMI_EINVAL.  The result is written to DEVICE memory (*maxColLengthDev, one uint32 the caller owns); the
 * kernels are queued on the null stream (so the call is ordered against every blocking stream, and cannot itself be recorded
 * into a graph) and the call returns without waiting for them; steps still queued in a runner are not run first (gennmi_flush
 * does that).  All calls on one GPU share
 * the array: calls that overlap on one GPU (from several threads or streams) race. */
#define GENNMI_STATIC_MAX_TARGETS (1u << 20)
int gennmi_max_col_length_static(uint32_t numSrcNeurons, uint32_t numTrgNeurons, uint32_t rowStride,
                                 const uint32_t *rowLength, const uint32_t *ind, uint32_t *maxColLengthDev);

/* updateSynapses(t)  backendCUDAHIP.cc:548-589: dendritic-delay pointer advance, presynaptic
 * update, postsynaptic update.  updateNeurons(t, recordingTimestep)  backendCUDAHIP.cc:386-420:
 * spike-queue reset and neuron update.  Asynchronous on the runner's stream. */
int gennmi_update_synapses(gennmi_runner *runner, float t);
int gennmi_update_neurons(gennmi_runner *runner, float t, uint32_t recordingTimestep);
/* updateSynapses(t) + updateNeurons(t, recordingTimestep) as one call, which lets delay networks take the
 * single-launch plan; a generated runner whose stepTime() body is fixed by generateRunner.cc:270-299 defers
 * updateSynapses and calls this from updateNeurons. */
int gennmi_step(gennmi_runner *runner, float t, uint32_t recordingTimestep);
/* stepTime(timestep, numRecordingTimesteps)  generateRunner.cc:270-299 */
int gennmi_step_time(gennmi_runner *runner, unsigned long long timestep, unsigned long long numRecordingTimesteps);
/* numSteps consecutive stepTime calls starting at `timestep` without a host round trip per step (no counterpart
 * in the reference, which launches 4-7 kernels per step from the host): one launch that keeps the network resident
 * on the chip where the runner's plan allows it (see gennmi_runner_get_info), else replays of a captured HIP graph
 * of 100 steps.  Either way the arrays are left as numSteps calls of gennmi_step_time would leave them. */
int gennmi_run_steps(gennmi_runner *runner, unsigned long long timestep, unsigned long long numSteps,
                     unsigned long long numRecordingTimesteps);
/* Step queue (no counterpart in the reference).  A caller that advances the model one gennmi_step() at a time -- the
 * reference's Runtime::stepTime() does, runtime.cc:686-697 -- pays one launch per step, while a runner on the resident
 * plan can take many steps in one launch.  With maxSteps > 0, gennmi_step() on such a runner only notes the step;
 * the noted steps are executed, as one launch where the plan allows it, before anything can observe the difference:
 * by every entry point of this library that reads, writes or frees device memory, synchronises, reads counters or
 * steps by another route, and when maxSteps steps are waiting.  Results are those of unqueued stepping; errors of a
 * queued step are reported by the call that executes it.  Runners on other plans, and runners with timing enabled,
 * step at once as before.  maxSteps = 0 (the default) switches the queue off after executing what it holds. */
int gennmi_runner_set_step_queue(gennmi_runner *runner, uint32_t maxSteps);
/* stepTimeFinalise: blocks until everything queued has finished and reports device-side
 * failures (backendCUDAHIP.cc:1400-1411). */
int gennmi_runner_synchronize(gennmi_runner *runner);

/* Timers: neuronUpdateTime / presynapticUpdateTime / postsynapticUpdateTime of generateRunner.cc:161-174,
 * in seconds, accumulated with HIP events while enabled (backendCUDAHIP.cc:36-76, 1479-1504).  While timing is enabled
 * every step is launched on its own, kernel by kernel (gennmi_run_steps included: no resident launch, no graph replay),
 * so that each kernel has an event pair around it.  A single-launch step (see gennmi_runner_get_info) is one kernel that
 * holds the neuron update and the presynaptic update of the previous step's spikes: its duration is reported as
 * neuronUpdateTime and presynapticUpdateTime stays 0 for such a runner. */
int gennmi_runner_set_timing(gennmi_runner *runner, int enabled);
int gennmi_runner_get_times(gennmi_runner *runner, double *neuronUpdateTime, double *presynapticUpdateTime,
                            double *postsynapticUpdateTime);
/* Launch counts and summed HIP-event durations (seconds) since the runner was created, measured while timing is
 * enabled: stats = {presynaptic launches, seconds, neuron launches, seconds, postsynaptic launches, seconds,
 * single-launch steps, seconds}.  Events are recorded on the runner's stream around every kernel and only read
 * (after one synchronisation) when statistics are requested, so timed stepping does not idle the device. */
int gennmi_runner_kernel_stats(gennmi_runner *runner, double stats[8]);
/* Two HIP events on the runner's stream: mark(0) before and mark(1) after a region of queued work, then
 * elapsed() = device time between them (blocks until mark 1 has completed).  This is the Timer of
 * backendCUDAHIP.cc:36-76 for a caller-chosen region, e.g. a whole gennmi_run_steps replay. */
int gennmi_runner_stream_mark(gennmi_runner *runner, int which);
int gennmi_runner_stream_elapsed(gennmi_runner *runner, double *seconds);
/* Launch plan chosen by gennmi_runner_finalise: bit 1 of info[0] is set if gennmi_run_steps keeps the network resident on
 * the chip (many steps per launch: batch 1, static SPARSE projections with ascending rows between LIF / Izhikevich
 * populations, all tiles of 256 neurons resident at once, and room in device memory for a per-(row, tile) table of 32 bytes
 * per entry and a second, 8-byte-per-synapse copy of the projections, both kept up to date with writes made through this
 * library; GENNMI_RESIDENT=0 disables it); bit 0 if a whole timestep is one launch (all projections go
 * through a dendritic-delay ring; synapses with d % D == 0 are then delivered by the spiking neuron one launch
 * earlier, into the slot read in the next step — the visible difference is the content of that one ring slot
 * between steps; GENNMI_FUSED_STEP=0 in the environment keeps the reference's placement); bit 2 if the neuron update
 * takes several neurons per lane (networks that need more than one round of resident work-groups and use only plain groups;
 * GENNMI_NEURON_BULK=0 forbids it, 2 / 4 / 8 force that many); bit 3: ordered accumulation; bit 4 if the scatter path, the
 * tile path and (bit 5) the postsynaptic passes of a step share one launch (projections with a tile path, or plastic ones
 * whose postsynaptic pass is paired with the presynaptic one: a synapse both of whose ends fired gets both rules from the
 * thread of the presynaptic pass, in the reference's order, and the postsynaptic pass leaves that row alone;
 * GENNMI_COMBINED=0 keeps a launch per kernel, GENNMI_PAIRED_LEARN=0 the reference's two passes); bit 6 if the busy steps
 * of a Toeplitz Conv2D projection run on the matrix cores (the layer as a GEMM over the source's spike bitmap in fp32 MFMA:
 * same products, sums in another order than the event-driven kernels'; GENNMI_CONV_MFMA=0 keeps those); info[1..3] = blocks of
 * the neuron, presynaptic and postsynaptic kernels.  The reference logs the analogous choice of presynaptic
 * strategy (backendSIMT.cc:736). */
int gennmi_runner_get_info(gennmi_runner *runner, uint32_t info[4]);
/* Synaptic events processed so far, summed over presynaptic groups (device counter). */
int gennmi_runner_event_count(gennmi_runner *runner, unsigned long long *events);


/* ---------------------------------------------------------------------------------------------
 * Generated kernels behind this boundary.  For model code the device library does not implement, the backend
 * generates gfx950 device code (one code object per module of the runner, built with `hipcc --genco` and embedded in
 * the module's object file); the runner itself stays host C++ and loads and launches that code through the calls
 * below.  This is what inline `kernel<<<grid, block, 0, stream>>>(...)` launches, hipEventRecord pairs and
 * hipGetLastError checks are in the reference's generated runner (src/genn/genn/code_generator/backendCUDAHIP.cc:386-420
 * genNeuronUpdate, :548-589 genSynapseUpdate, :750-856 genCustomUpdate, :1479-1504 genTimer).
 *
 * A program owns a stream (the runner's, when it is created beside one), the code objects, a device error flag that
 * its kernels raise when a bounded wait expires, timers, and the sequence of launches that makes up each phase of a
 * timestep (GENNMI_PHASE_SYNAPSES = updateSynapses, GENNMI_PHASE_NEURONS = updateNeurons).  Every kernel takes a
 * gennmi_launch_header_t as its first argument and the launch's own argument block as its second; the header tells it
 * where the values of its step are: in `inlineEntry` (steps[] == NULL: a launch made when it was asked for) or in
 * steps[k] (device memory: a launch replayed from a captured HIP graph, whose arguments cannot change from replay to
 * replay).  With stepQueueLength > 0 gennmi_program_update() only notes the call; noted calls run, from a graph of the
 * whole queue when it is full and the phases came in the order the graph was captured for, before anything can observe
 * the difference (every entry point of this library that reads, writes or frees device memory, synchronises or
 * launches by another route executes them first).
 * ------------------------------------------------------------------------------------------- */
typedef struct gennmi_program gennmi_program;
typedef struct gennmi_step_entry
{
    double t;                       /* simulation time of the step (converted to the model's time type in the kernel) */
    unsigned long long step;        /* calls of this phase so far: the step counter of counter-based random numbers */
    uint32_t recordingTimestep;     /* row of the recording buffers */
    uint32_t tag;                   /* differs from one call of a phase to the next and is never 0 (tagged look-back words) */
} gennmi_step_entry_t;
typedef struct gennmi_launch_header
{
    const gennmi_step_entry_t *steps;   /* device table of the queued calls, or NULL */
    uint32_t k;                         /* index into steps */
    uint32_t spinLimit;                 /* polls a work-group waits for another one before it raises the error flag */
    gennmi_step_entry_t inlineEntry;    /* used when steps == NULL */
} gennmi_launch_header_t;
enum { GENNMI_PHASE_SYNAPSES = 0, GENNMI_PHASE_NEURONS = 1, GENNMI_NUM_PHASES = 2 };
#define GENNMI_MAX_LAUNCH_ARG_BYTES 3072u
#define GENNMI_MAX_TIMERS 64

/* `runner` may be NULL (a model whose step runs on generated kernels only); otherwise the program shares the runner's
 * stream, so that its launches are ordered against the runner's.  stepQueueLength = 0: every call launches at once. */
int gennmi_program_create(gennmi_program **program, gennmi_runner *runner, uint32_t stepQueueLength);
int gennmi_program_destroy(gennmi_program *program);
/* hipModuleLoadData / hipModuleGetFunction: `image` is a gfx950 code object in host memory (it is copied) */
int gennmi_program_load_module(gennmi_program *program, const void *image, size_t bytes, uint32_t *module);
int gennmi_program_get_kernel(gennmi_program *program, uint32_t module, const char *name, uint32_t *kernel);
/* the device word the program's kernels raise (atomicOr) when a bounded wait expires; reported as GENNMI_EDEVICE by
 * gennmi_program_synchronize and by the next gennmi_synchronize / gennmi_memcpy_from_device that follows the launches */
int gennmi_program_error_flag(gennmi_program *program, uint32_t **deviceFlag);
/* Appends a launch to a phase's sequence: kernel<<<dim3(gridX, gridY), dim3(blockX), 0, stream>>>(header, args).
 * `args` (argBytes <= GENNMI_MAX_LAUNCH_ARG_BYTES, 8-byte aligned layout) is copied.  `timer` (0 ..
 * GENNMI_MAX_TIMERS-1, or -1) names the timer that accumulates the launch's duration while timing is enabled.
 * gennmi_program_clear_phases forgets every sequence (and the captured graph). */
int gennmi_program_add_launch(gennmi_program *program, int phase, uint32_t kernel, uint32_t gridX, uint32_t gridY, uint32_t blockX,
                              const void *args, size_t argBytes, int timer);
int gennmi_program_clear_phases(gennmi_program *program);
/* updateSynapses(t) / updateNeurons(t, recordingTimestep) of a runner on generated kernels: runs (or notes) the
 * phase's launches.  Replaces the launch sequences of backendCUDAHIP.cc:386-420 and :548-589. */
int gennmi_program_update(gennmi_program *program, int phase, double t, uint32_t recordingTimestep);
/* One launch now, after everything noted has run (custom updates: update<Group>(), backendCUDAHIP.cc:750-856).
 * `step`: the counter handed to the kernel in its header's inlineEntry. */
int gennmi_program_launch(gennmi_program *program, uint32_t kernel, uint32_t gridX, uint32_t gridY, uint32_t blockX,
                          const void *args, size_t argBytes, double t, unsigned long long step, int timer);
/* blocks until the program's stream is idle; GENNMI_EDEVICE if a kernel raised the error flag */
int gennmi_program_synchronize(gennmi_program *program);
/* Timers (genTimer, backendCUDAHIP.cc:1479-1504): while enabled, nothing is queued or replayed from a graph and every
 * launch has a HIP event pair around it; get_time returns the seconds accumulated by a timer since creation. */
int gennmi_program_set_timing(gennmi_program *program, int enabled);
int gennmi_program_get_time(gennmi_program *program, int timer, double *seconds);
/* info = {calls of gennmi_program_update executed so far, of which replayed from a captured graph, launches made, graphs captured} */
int gennmi_program_get_info(gennmi_program *program, unsigned long long info[4]);

#ifdef __cplusplus
}
#endif
#endif
