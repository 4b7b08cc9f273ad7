/* salt_gpu_mi355_engine.h -- the engine-facing half of libsalt_gpu_mi355.so.
 *
 * SALT links exactly one physical backend object behind include/salt/gpu.h
 * (reference Makefile:24-47).  This header restates, for the quantized decode
 * path, the entry points and plain-C structures of that interface with the
 * same names, argument order and layouts, so the library can be linked in
 * place of the reference's gpu_hip.o.  Everything is host-pointer based and
 * synchronous unless defer mode is on; 0 = done, -1 = unavailable or failed
 * (reference gpu.h:23-25).  Entry points of gpu.h that are not on this path
 * (q8, bf16, attention, exact cells, tensor program, dispatch table, legacy
 * trunk/pool maps) are exported too and answer exactly like the reference's
 * null backend (src/gpu_stub.c), so the link resolves and the engine falls
 * back to its CPU kernels for them.
 *
 * Where the weights live.  The engine describes host byte ranges (mmap'ed
 * model files, expert cache slots) and names tensors inside them by a stable
 * key.  On an MI355X every activated range is copied once into HBM (288 GB
 * holds every supported model whole) and kernels only ever read the HBM copy;
 * the engine's host pointers are turned into device addresses by their offset
 * from the described base.  Expert cache seats are filled through the
 * residency operations (engine read callback -> pinned staging -> HBM seat).
 */
#ifndef SALT_GPU_MI355_ENGINE_H
#define SALT_GPU_MI355_ENGINE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- lifecycle, modes, statistics --------------------------------------- */

int salt_gpu_init(void);                          /* reference gpu.h:26 */
int salt_gpu_free(void);                          /* reference gpu.h:27; -1 while a residency arena is live */
int salt_gpu_cuda_present(void);                  /* reference gpu.h:168; always 0 */
int salt_gpu_rocm_present(void);                  /* reference gpu.h:170; always 1 */
int salt_gpu_pageable_mmap_active(void);          /* reference gpu.h:173; always 0 */
void salt_gpu_set_mapped_only(int on);            /* reference gpu.h:99 */
int salt_gpu_mapped_only(void);                   /* reference gpu.h:100 */
int salt_gpu_set_defer(int on);                   /* reference gpu.h:190; turning it off syncs */
int salt_gpu_defer(void);                         /* reference gpu.h:191 */
int salt_gpu_sync(void);                          /* reference gpu.h:192; publishes deferred outputs */

typedef struct SaltGpuBatchStats {                /* reference gpu.h:102-109 */
    uint64_t arena_batches;
    uint64_t trunk_batches;
    uint64_t expert_layer_batches;
    uint64_t mapped_only_misses;
    uint64_t direct_output_batches;
    uint64_t direct_output_jobs;
} SaltGpuBatchStats;

typedef struct SaltGpuBatchStatsV2 {              /* reference gpu.h:111-132 */
    uint64_t arena_batches;
    uint64_t trunk_batches;
    uint64_t expert_layer_batches;
    uint64_t mapped_only_misses;
    uint64_t direct_output_batches;
    uint64_t direct_output_jobs;
    uint64_t nvfp4_logical_packed_weight_bytes;
    uint64_t nvfp4_logical_weight_scale_bytes;
    uint64_t nvfp4_activation_input_bytes;
    uint64_t nvfp4_activation_qdq_bytes;
    uint64_t nvfp4_projection_output_bytes;
    uint64_t nvfp4_kernel_launches;
    uint64_t nvfp4_completion_fences;
    uint64_t nvfp4_h2d_ns;
    uint64_t nvfp4_qdq_ns;
    uint64_t nvfp4_projection_ns;
    uint64_t nvfp4_d2h_ns;
    uint64_t q4_weight_stationary_batches;
} SaltGpuBatchStatsV2;

void salt_gpu_batch_stats_get(SaltGpuBatchStats *stats);                        /* reference gpu.h:134 */
int salt_gpu_batch_stats_get_v2(SaltGpuBatchStatsV2 *stats, size_t stats_size); /* reference gpu.h:135 */

typedef struct SaltGpuStartupRequirements {       /* reference gpu.h:431-440 */
    uint64_t fixed_device_bytes;
    uint64_t fixed_pinned_host_bytes;
    uint64_t descriptor_bytes;
    uint64_t device_copied_weight_bytes;
    uint32_t max_output_floats;
    uint32_t max_batch_jobs;
    uint32_t shared_buffer_slots;
    uint32_t reserved;
} SaltGpuStartupRequirements;
/* reference gpu.h:443; pure query, no initialisation */
int salt_gpu_startup_requirements(SaltGpuStartupRequirements *requirements, size_t requirements_size);

/* ---- weight resources: identity, addressability, tensor keys ------------- */

typedef enum SaltGpuWeightAddressability {        /* reference gpu.h:411-416 */
    SALT_GPU_WEIGHT_ADDRESS_AUTO = 0,
    SALT_GPU_WEIGHT_ADDRESS_BOUNDED_WINDOW = 1,
    SALT_GPU_WEIGHT_ADDRESS_REGISTERED_PERSISTENT = 2,
    SALT_GPU_WEIGHT_ADDRESS_PAGEABLE = 3
} SaltGpuWeightAddressability;

typedef struct SaltGpuWeightResourceUsage {       /* reference gpu.h:418-429 */
    uint64_t described_bytes;
    uint64_t registered_bytes;
    uint64_t pageable_bytes;
    uint64_t active_window_bytes;
    uint64_t peak_window_bytes;
    uint64_t device_copied_weight_bytes;
    uint32_t described_resources;
    uint32_t active_resources;
    uint32_t active_windows;
    uint32_t reserved;
} SaltGpuWeightResourceUsage;

/* reference gpu.h:450-460, 465-469, 480.  describe records a host range;
 * activate (AUTO or REGISTERED_PERSISTENT) copies it to HBM once;
 * BOUNDED_WINDOW copies only the windows later bound; PAGEABLE is refused.
 * pool_bind (reference gpu_hip.cpp:4208-4217) turns an active, window-addressed
 * resource with nothing bound into a component pool: only the byte ranges its
 * registered tensors occupy become resident (merged, 4096-byte granules of the
 * resource offset), either as the permanent spans of the residency arena or,
 * when the engine runs no arena, in HBM allocations made at the next
 * salt_gpu_sync.  A pool that is laid out or resident no longer grows. */
int salt_gpu_weight_resource_describe(uint32_t kind, uint32_t resource_id, const void *base, size_t nbytes);
int salt_gpu_weight_resource_activate(uint32_t kind, uint32_t resource_id, SaltGpuWeightAddressability policy);
int salt_gpu_weight_resource_pool_bind(uint32_t kind, uint32_t resource_id);
int salt_gpu_weight_resource_deactivate(uint32_t kind, uint32_t resource_id);
int salt_gpu_weight_resource_usage(SaltGpuWeightResourceUsage *usage, size_t usage_size);
int salt_gpu_weight_resource_bind(uint32_t kind, uint32_t resource_id, const void *base, size_t nbytes);
int salt_gpu_weight_window_bind(uint32_t kind, uint32_t resource_id, uint64_t offset, size_t nbytes);
int salt_gpu_weight_window_unbind(uint32_t kind, uint32_t resource_id);
int salt_gpu_weight_resource_unbind(uint32_t kind, uint32_t resource_id);
/* reference gpu.h:470-479: name a tensor inside a described resource */
int salt_gpu_weight_resource_slot(uint32_t kind, uint32_t resource_id, const void *key, const uint32_t *vals,
                                  const uint16_t *scales, const uint16_t *biases, int bits, int R, int C);
int salt_gpu_nvfp4_resource_slot(uint32_t kind, uint32_t resource_id, const void *key,
                                 const uint8_t *weight_packed, const uint8_t *weight_scales,
                                 const float *weight_global_scale, const float *input_global_scale, int R, int C);
/* reference gpu.h:395-409: command-scoped expert layer resources */
int salt_gpu_resident_slot(const void *key, const uint32_t *vals, const uint16_t *scales,
                           const uint16_t *biases, int R, int C);
int salt_gpu_expert_resource_bind(uint32_t resource_id, const void *base, size_t nbytes);
int salt_gpu_expert_resource_slot(uint32_t resource_id, const void *key, const uint32_t *vals,
                                  const uint16_t *scales, const uint16_t *biases, int R, int C);
int salt_gpu_expert_resource_unbind(uint32_t resource_id);

/* ---- shared buffers ------------------------------------------------------ */

typedef struct SaltGpuSharedBuffer {              /* reference gpu.h:198-202 */
    void *contents;      /* host address */
    size_t nbytes;
    void *backend;       /* the same memory as the device sees it */
} SaltGpuSharedBuffer;
int salt_gpu_shared_buffer_alloc(SaltGpuSharedBuffer *buffer, size_t nbytes);   /* reference gpu.h:204 */
int salt_gpu_shared_buffer_free(SaltGpuSharedBuffer *buffer);                   /* reference gpu.h:205 */

/* ---- affine Q4 compute ---------------------------------------------------- */

/* reference gpu.h:34: one matvec, weights given by host pointers */
int salt_gpu_q4_matvec(const uint32_t *vals, const uint16_t *scales, const uint16_t *biases, int R, int C,
                       const float *x, float *y);
/* reference gpu.h:83: njobs matvecs sharing C, one dispatch */
int salt_gpu_q4_batch(const uint32_t *const *vals, const uint16_t *const *scales, const uint16_t *const *biases,
                      const float *const *xs, float *const *ys, const void *const *ids, const int *Rj, int C,
                      int njobs);
/* reference gpu.h:388: one weight, B contiguous tokens */
int salt_gpu_proj_batch(const uint32_t *vals, const uint16_t *scales, const uint16_t *biases, int R, int C, int B,
                        const float *const *xs, float *const *ys, const void *id);
/* reference gpu.h:354-368: asynchronous, writes straight into a shared buffer, published by salt_gpu_sync */
int salt_gpu_proj_batch_indexed(const uint32_t *vals, const uint16_t *scales, const uint16_t *biases, int R, int C,
                                int B, int first_job, int job_count, const float *xs, SaltGpuSharedBuffer *output,
                                size_t y_float_offset, const void *id);
int salt_gpu_proj_batch_indexed_exact_views(const uint32_t *vals, const uint16_t *scales, const uint16_t *biases,
                                            int R, int C, int B, int first_job, int job_count, const float *xs,
                                            SaltGpuSharedBuffer *output, size_t y_float_offset, const void *id);

typedef struct SaltGpuMoeExpert {                 /* reference gpu.h:276-295 */
    const uint32_t *gate_vals;
    const uint16_t *gate_scales;
    const uint16_t *gate_biases;
    const void *gate_id;
    const uint32_t *up_vals;
    const uint16_t *up_scales;
    const uint16_t *up_biases;
    const void *up_id;
    const uint32_t *down_vals;
    const uint16_t *down_scales;
    const uint16_t *down_biases;
    const void *down_id;
    int group;                    /* token rows routed to this expert */
    int resource_slot;            /* expert-cache seat, or -1 */
    uint64_t logical_resource_id; /* layer * n_experts + expert */
} SaltGpuMoeExpert;

/* reference gpu.h:320-329: gate, up, gelu*up, down for `count` experts; rows
 * of inputs/outputs grouped by expert in the order given; the weighted
 * reduction stays with the engine.  The _selected form takes its four buffers
 * as shared buffers and the device reads `inputs` where they lie, without a
 * snapshot: they must stay unchanged until the call returns or, in deferred
 * mode (salt_gpu_set_defer), until salt_gpu_sync() has returned. */
int salt_gpu_q4_moe_chain(const SaltGpuMoeExpert *experts, int count, int hidden, int routed, const float *inputs,
                          float *outputs, float *gate_scratch, float *up_scratch, size_t scratch_float_capacity);
int salt_gpu_q4_moe_chain_selected(const SaltGpuMoeExpert *experts, int count, int hidden, int routed,
                                   const float *inputs, float *outputs, float *gate_scratch, float *up_scratch,
                                   size_t scratch_float_capacity);

typedef struct SaltGpuSelectedProjectionJob {     /* reference gpu.h:297-309 */
    const uint32_t *vals;
    const uint16_t *scales;
    const uint16_t *biases;
    const void *id;
    const float *inputs;
    float *outputs;
    int rows;
    int cols;
    int batch;
    int resource_slot;
    uint64_t logical_resource_id;
} SaltGpuSelectedProjectionJob;
/* reference gpu.h:314 */
int salt_gpu_q4_selected_shared(const SaltGpuSelectedProjectionJob *jobs, int job_count, SaltGpuSharedBuffer *arena);

/* reference gpu.h:335-347: expert-cache seats */
int salt_gpu_selected_resources_prepare(int capacity, int logical_capacity);
int salt_gpu_selected_resource_bind(int slot, uint64_t logical_resource_id, const void *base, size_t nbytes,
                                    const void *payload);
int salt_gpu_selected_resource_bind_resident(int slot, uint64_t logical_resource_id, const void *payload,
                                             size_t nbytes, uintptr_t device_address, uint64_t generation);
int salt_gpu_selected_resources_fence(void);
int salt_gpu_selected_resource_unbind(int slot, uint64_t logical_resource_id);

/* ---- NVFP4 compute --------------------------------------------------------- */

/* reference gpu.h:44-59 */
int salt_gpu_nvfp4_qdq(const float *input, int C, float input_global_scale, uint8_t *packed, uint8_t *scales,
                       float *dequant);
int salt_gpu_nvfp4_matvec(const void *key, int R, int C, const float *input, float *output);
int salt_gpu_nvfp4_matvec_batch(const void *key, int R, int C, int B, const float *inputs, float *outputs);
int salt_gpu_nvfp4_batch(const void *const *keys, const float *const *inputs, float *const *outputs,
                         const int *batches, int R, int C, int njobs);
int salt_gpu_nvfp4_mixed_batch(const void *const *keys, const float *const *inputs, float *const *outputs,
                               const int *batches, const int *rows, int C, int njobs);

/* ---- device residency (reference include/salt/gpu_residency.h:25-89, 149) -- */

typedef struct SaltGpuResourceRef {               /* reference gpu_resource.h:16-22 */
    uint32_t kind;
    uint32_t resource_id;
    uint64_t value_offset;
    uint64_t scale_offset;
    uint64_t bias_offset;
} SaltGpuResourceRef;

typedef struct SaltGpuResidencyPlan {
    uint64_t device_budget_bytes;
    uint64_t permanent_bytes;
    uint64_t slot_base_offset;
    uint64_t slot_bytes;
    uint64_t staging_bytes;
    uint32_t slot_count;
    uint32_t staging_count;
    uint32_t device_alignment;
    uint32_t flags;
} SaltGpuResidencyPlan;

typedef int (*SaltGpuResidencyReadFn)(void *context, uint64_t source_offset, void *destination, size_t nbytes);

typedef struct SaltGpuResidencySource {
    SaltGpuResourceRef resource;
    uint64_t logical_resource_id;
    uint64_t source_offset;
    uint64_t nbytes;
    SaltGpuResidencyReadFn read;
    void *read_context;
} SaltGpuResidencySource;

typedef struct SaltGpuResidencyPermanentLayout {
    uint64_t permanent_bytes;
    uint64_t maximum_span_bytes;
    uint32_t span_count;
    uint32_t alignment;
} SaltGpuResidencyPermanentLayout;

typedef struct SaltGpuResidencyPermanentSpan {
    SaltGpuResidencySource source;
    uint64_t device_offset;
} SaltGpuResidencyPermanentSpan;

#define SALT_GPU_RESIDENCY_ABI_VERSION 1u

/* The engine's slot state machine (reference src/gpu_residency.c) drives these:
 * create an HBM arena plus pinned staging, hand out staging for the engine's
 * read callback, copy staging -> seat asynchronously (populate), report
 * completion (poll), translate offsets to device addresses (resolve), drain a
 * seat before reuse (retire), and tear down (destroy).  The permanent_* ops
 * (reference gpu_hip.cpp:3429-3571) enumerate the regions of the component pool
 * as spans at 256-byte aligned offsets in front of the seats, give the engine a
 * read callback for each, copy its staged chunks in order (permanent_copy is
 * complete on return) and, once every span is full, make the tensors inside
 * resolvable (permanent_publish).  Without a pool-bound resource that holds
 * tensors permanent_layout returns -1; destroy takes the spans with the arena. */
typedef struct SaltGpuResidencyBackendOps {
    uint32_t abi_version;
    size_t ops_size;
    int (*create)(void *context, const SaltGpuResidencyPlan *plan);
    int (*staging)(void *context, uint32_t staging_slot, void **address, size_t *capacity);
    int (*populate)(void *context, uint32_t physical_slot, uint64_t device_offset, uint32_t staging_slot,
                    size_t nbytes, uint64_t ticket);
    int (*poll)(void *context, uint32_t physical_slot, uint64_t ticket, int *complete);
    int (*resolve)(void *context, uint64_t device_offset, size_t nbytes, uintptr_t *address);
    int (*retire)(void *context, uint32_t physical_slot, uint64_t generation);
    int (*destroy)(void *context);
    int (*permanent_layout)(void *context, SaltGpuResidencyPermanentLayout *layout, size_t layout_size);
    int (*permanent_span)(void *context, uint32_t span_index, SaltGpuResidencyPermanentSpan *span,
                          size_t span_size);
    int (*permanent_copy)(void *context, uint32_t span_index, uint64_t device_offset, uint32_t staging_slot,
                          size_t nbytes, uint64_t ticket);
    int (*permanent_publish)(void *context);
} SaltGpuResidencyBackendOps;
const SaltGpuResidencyBackendOps *salt_gpu_residency_backend_ops(void);   /* reference gpu_residency.h:149 */

/* ---- 8-bit affine router gates and the bf16 head --------------------------- */

/* 8-bit tensors are registered with salt_gpu_weight_resource_slot(bits = 8).  One left-to-right chain per row
 * (reference src/kernels.c:343-370): bit-exact. */
int salt_gpu_q8_matvec(const uint32_t *vals, const uint16_t *scales, const uint16_t *biases, int R, int C,
                       const float *x, float *y);                               /* reference gpu.h:37 */
int salt_gpu_q8_batch(const uint32_t *const *vals, const uint16_t *const *scales, const uint16_t *const *biases,
                      const float *const *xs, float *const *ys, const void *const *ids, const int *Rj, int C,
                      int njobs);                                                /* reference gpu.h:89 */
/* C must be a multiple of 8 and the key registered (reference gpu_hip.cpp:4414-4443, 4591-4622); eight chains per row
 * in the order of src/kernels.c:139-174: bit-exact. */
int salt_gpu_bf16_resource_slot(uint32_t kind, uint32_t resource_id, const void *key, const uint16_t *weights,
                                int R, int C);                                   /* reference gpu.h:60 */
int salt_gpu_bf16_matvec(const void *key, int R, int C, const float *input, float *output);   /* reference gpu.h:63 */

/* ---- fp32 cells over shared buffers ----------------------------------------- */

typedef enum SaltGpuExactCellKind {               /* reference gpu.h:211-218 */
    SALT_GPU_EXACT_RMSNORM = 1,
    SALT_GPU_EXACT_TOPK = 2,
    SALT_GPU_EXACT_RESIDUAL_POSTNORM = 3,
    SALT_GPU_EXACT_PARALLEL_COMBINE = 4,
    SALT_GPU_EXACT_SOFTCAP = 5,
    SALT_GPU_EXACT_ROUTER_INPUT = 6
} SaltGpuExactCellKind;

typedef struct SaltGpuExactCell {                 /* reference gpu.h:224-232 */
    SaltGpuExactCellKind kind;
    SaltGpuSharedBuffer *views[8];   /* per kind as in reference gpu_hip.cpp:5299-5400 */
    size_t offsets[8];               /* element offsets (floats; ints for the selection of TOPK) */
    uint32_t n;
    uint32_t aux;
    float eps;
    float scalar;
} SaltGpuExactCell;

/* The cells run in order on the device; one completion for the sequence.  -1 when a cell meets a non-finite input or
 * result (that cell and every later one then publish nothing) or a view lies outside its buffer. */
int salt_gpu_exact_cells(const SaltGpuExactCell *cells, int count);              /* reference gpu.h:234 */

/* ---- whole-mapping conveniences ------------------------------------------- */

/* One mapped trunk range at a time, copied to HBM as trunk resource 0 (reference gpu_metal.m:1533-1536); unmap
 * releases it (reference gpu_hip.cpp:5180).  pool_map is expert-layer resource 0 (reference gpu_metal.m:1633-1642). */
int salt_gpu_resident_trunk_map(const void *base, size_t nbytes);                /* reference gpu.h:180 */
int salt_gpu_resident_trunk_unmap(void);                                         /* reference gpu.h:183 */
int salt_gpu_resident_pool_map(const void *base, size_t nbytes);                 /* reference gpu.h:484 */

/* ---- outside the quantized decode path: answered like the null backend ---- */

struct SaltGpuDispatch;
struct SaltTextGpuProgramOps;
/* left to the CPU, as in the reference's ROCm backend (gpu_hip.cpp:4624-4628) */
int salt_gpu_bf16_matvec_batch(const void *key, int R, int C, int B, const float *inputs, float *outputs);
const struct SaltGpuDispatch *salt_dispatch_get(void);                           /* reference gpu.h:163 */
const struct SaltTextGpuProgramOps *salt_gpu_tensor_program_ops(void);           /* reference gpu.h:209 */
/* reference gpu.h:239-274: prefill attention, KV mirror and Q/K/V transform */
int salt_gpu_attention_batch(int full_attention, int n_heads, int n_kv_heads, int head_dim, int window,
                             const SaltGpuSharedBuffer *queries, size_t query_float_offset,
                             const SaltGpuSharedBuffer *kv, size_t key_float_offset, size_t value_float_offset,
                             int start_position, int batch, int query_stride, int kv_stride,
                             SaltGpuSharedBuffer *outputs, size_t output_float_offset,
                             SaltGpuSharedBuffer *score_workspace, size_t score_float_offset, size_t score_stride,
                             int score_task_capacity);
int salt_gpu_attention_prepare(const SaltGpuSharedBuffer *kv);
int salt_gpu_attention_bind_kv(size_t key_float_offset, size_t value_float_offset, int kv_stride);
int salt_gpu_attention_materialize(SaltGpuSharedBuffer *kv, int position, uint64_t *copied_bytes);
int salt_gpu_attention_import(SaltGpuSharedBuffer *kv, int position, uint64_t *copied_bytes);
int salt_gpu_attention_rewind(int position);
int salt_gpu_attention_transform(int n_heads, int n_kv_heads, int head_dim, int rope_dim, int start_position,
                                 int batch, int query_stride, int kv_stride, float eps,
                                 SaltGpuSharedBuffer *queries, size_t query_float_offset,
                                 SaltGpuSharedBuffer *keys, size_t key_float_offset,
                                 SaltGpuSharedBuffer *values, size_t value_float_offset, const float *q_weight,
                                 const float *k_weight, const float *cosines, const float *sines, int rope_pairs,
                                 SaltGpuSharedBuffer *kv, size_t key_cache_float_offset,
                                 size_t value_cache_float_offset);

#ifdef __cplusplus
}
#endif

#endif /* SALT_GPU_MI355_ENGINE_H */
