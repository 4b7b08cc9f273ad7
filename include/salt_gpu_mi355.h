/* salt_gpu_mi355.h -- C ABI of libsalt_gpu_mi355.so, the MI355X (gfx950)
 * backend for SALT's quantized decode path.
 *
 * Two groups of entry points:
 *
 *  1. The engine's physical-backend ABI for this path.  These carry the names
 *     and signatures of the reference's include/salt/gpu.h so that linking this
 *     library in place of the reference's gpu_hip.o / gpu_stub.o needs no
 *     engine change; each declaration cites the reference lines it replaces.
 *     All pointers are host pointers owned by the caller; 0 = done, -1 =
 *     unavailable or failed (reference gpu.h:23-25).  They are declared in
 *     salt_gpu_mi355_engine.h, which this header includes.
 *
 *  2. Device-resident entry points (salt_mi355_*): the same operations on
 *     buffers that already live in HBM, launched on a caller-supplied HIP
 *     stream.  The engine-facing calls are thin host wrappers around these.
 *     They have no counterpart in the reference ABI, whose every call moves
 *     activations across the host boundary; harnesses that keep data on the
 *     device (the benchmark, the parity tests, a future whole-layer program)
 *     call them directly.
 *
 * Plain C, no HIP or torch types: a stream is passed as void* (hipStream_t,
 * NULL = the null stream) and device memory as void* / typed pointers.
 * The library is not thread-safe; like the reference backends it expects one
 * owner thread (reference gpu_hip.cpp keeps global state without locks).
 */
#ifndef SALT_GPU_MI355_H
#define SALT_GPU_MI355_H

#include <stddef.h>
#include <stdint.h>

#include "salt_gpu_mi355_engine.h"

#ifdef __cplusplus
extern "C" {
#endif

/* ---- lifecycle and diagnostics ---------------------------------------- */

/* Selects device 0, creates the library stream, and checks on the device that
 * the fp8 and fp4 converters decode the way the kernels assume.  Idempotent.
 * salt_gpu_init (reference gpu.h:26) calls this. */
int salt_mi355_init(void);
int salt_mi355_shutdown(void);
/* Last failure recorded by any entry point, for logs; never NULL. */
const char *salt_mi355_last_error(void);
/* Name and template arguments of the Q4 matvec kernel that the last launch used (for bench records); never NULL. */
const char *salt_mi355_last_kernel(void);
/* Raw decode tables measured at init: fp8[b] is what v_cvt_pk_f32_fp8 returns
 * for byte b; fp4[2*b], fp4[2*b+1] what v_cvt_scalef32_pk_f32_fp4 (scale 1)
 * returns for the low and high nibble of byte b.  Host arrays of 256 / 512. */
int salt_mi355_converter_tables(float *fp8, float *fp4);

/* ---- device memory and timing helpers for host harnesses --------------- */

void *salt_mi355_dev_alloc(size_t nbytes);
int salt_mi355_dev_free(void *device_ptr);
int salt_mi355_dev_upload(void *device_dst, const void *host_src, size_t nbytes);
int salt_mi355_dev_download(void *host_dst, const void *device_src, size_t nbytes);
int salt_mi355_dev_fill(void *device_dst, int byte_value, size_t nbytes);
/* The library's own stream (default priority), as a hipStream_t. */
void *salt_mi355_stream(void);
int salt_mi355_stream_sync(void *stream);
void *salt_mi355_event_create(void);
int salt_mi355_event_destroy(void *event);
int salt_mi355_event_record(void *event, void *stream);
/* Waits for `stop`, then returns the milliseconds between the two events. */
int salt_mi355_event_elapsed_ms(void *start, void *stop, float *ms);
/* Policy, off by default: with it the engine entry points (salt_gpu_q4_matvec,
 * salt_gpu_q4_batch, salt_gpu_proj_batch*, salt_gpu_q4_moe_chain*,
 * salt_gpu_nvfp4_matvec / _batch of up to four tokens) run the tolerance-class
 * kernels of salt_mi355_q4_jobs_t_dev / salt_mi355_nvfp4_matvec_t_dev instead of
 * the bit-exact ones: results then carry those entry points' stated bounds
 * and are no longer bit-identical to the reference CPU kernels.  Never read
 * from the environment: an engine opts in with this call (compare the
 * reference's own policy setters salt_gpu_set_mapped_only / salt_gpu_set_defer,
 * gpu.h:96-100, 190-192).  Returns the previous setting. */
int salt_mi355_set_tolerance_class(int enabled);

/* Stream capture for callers that replay a fixed sequence of the device-resident
 * entry points as one HIP graph.  Capturable: every *_dev entry point that takes
 * a status word and neither uploads a job table nor waits (the MoE decode step,
 * the feed-forward block, the cells, single-matrix matvecs, *_jobs_* launches
 * of up to 16 jobs: their records travel in the kernel arguments).  A *_jobs_*
 * call with more jobs copies a table to the device through a ring of pinned
 * buffers that it waits on and rewrites: under capture it is refused (-1) with
 * an error that says so.  begin starts a
 * capture on `stream`; end finishes it and returns an executable graph (NULL on
 * failure); launch replays it on `stream`. */
int salt_mi355_graph_begin(void *stream);
void *salt_mi355_graph_end(void *stream);
int salt_mi355_graph_launch(void *graph_exec, void *stream);
int salt_mi355_graph_destroy(void *graph_exec);
/* Measurement aid (no counterpart in the reference): one or two kernels with
 * empty bodies, launched one after the other on `stream` with the given
 * numbers of workgroups, threads per workgroup and bytes of dynamic LDS
 * (workgroups 0: that launch is left out).  What a step's launches cost with
 * nothing in them: the floor its arithmetic sits on. */
int salt_mi355_launch_skeleton_dev(int workgroups_a, int threads_a, int lds_bytes_a,
                                   int workgroups_b, int threads_b, int lds_bytes_b, void *stream);

/* ---- affine Q4 ("mlx4") matvec, device-resident ------------------------
 * Layout as the reference's salt_q4_matvec (kernels.h:117-130): u32 words of
 * eight nibbles, low nibble first, flat element index r*C + c; one bf16 scale
 * and one bf16 bias per 64 flat elements (biases may be NULL: bias 0).
 * ys[t*R + r] is bit-identical to the reference CPU row (kernels.c:220-250)
 * against xs[t*C ..].  B >= 1 tokens; weights are streamed once per group of
 * four tokens.  chains_per_lane: 0 = choose, or 8 / 4 / 2 (tuning knob). */
int salt_mi355_q4_matvec_dev(const void *vals, const void *scales, const void *biases,
                             int R, int C, int B, const float *xs, float *ys,
                             int chains_per_lane, void *stream);

/* Many matrices in one launch (the shape of reference salt_gpu_q4_batch,
 * gpu.h:83): job j multiplies its own R_j x C matrix with its own tokens.
 * `jobs` is a HOST array; the library copies it to the device on `stream`. */
typedef struct SaltMi355Q4Job {
    const void *vals;
    const void *scales;
    const void *biases;      /* may be NULL */
    const float *xs;         /* device, [tokens][C] */
    float *ys;               /* device, [tokens][rows] */
    int rows;
} SaltMi355Q4Job;
int salt_mi355_q4_jobs_dev(const SaltMi355Q4Job *jobs, int njobs, int C, int tokens,
                           int chains_per_lane, void *stream);
/* The down projections of a decode-shaped expert chain in one launch, without a launch for the activation: every
 * job has one token, and its activation row is gelu_tanh(g[i]) * u[i] (reference gemma4.c:80-83,
 * gemma4_text.c:7608-7649) where g = job.xs and u = job.xs + up_offset_floats, both [C] floats on the device.  C a
 * multiple of 64 up to 4096; pointers as the tiled kernel needs them (values 4-byte, scales and biases 2-byte
 * aligned), else -1.  ys[j] is bit-identical to salt_mi355_moe_activate_dev followed by salt_mi355_q4_jobs_dev. */
int salt_mi355_q4_jobs_activated_dev(const SaltMi355Q4Job *jobs, int njobs, int C, long long up_offset_floats,
                                     void *stream);
/* Tolerance-class decode matvec: the memory-bound kernel.  Same layouts and
 * shapes as salt_mi355_q4_matvec_dev / salt_mi355_q4_jobs_dev, but NOT
 * bit-identical to the reference row (kernels.c:220-250), whose 32-chain order
 * with four roundings per weight costs more vector instructions than the
 * memory system leaves time for.  Per 64-column scale group the kernel forms
 *   scale * sum_c q_c * x_c + bias * sum_c x_c
 * with the integer-by-activation sums exact (activations in block fixed point
 * of 31 bits below each group's largest magnitude) and a few fp32 roundings per
 * group.  Bound, per output:
 *   |y - y_ref| <= 2^-20 * sum_c (|q_c s| + 16 |s| + |b|) |x_c| + 1e-6.
 * A non-finite activation makes every output of its token non-finite (the
 * reference: the rows that touch it).  C a multiple of 64, at least 512, and
 * dword-aligned values take the streaming kernel; anything else runs on the
 * bit-exact kernels.  The reference has no counterpart (north star: "otherwise
 * within a stated max-abs/relative fp32 tolerance").
 *
 * Which bits a result has depends on the LAUNCH, not only on the matrix and
 * the activation: the column count, the number of tokens and the number of
 * 32-row blocks summed over all jobs of the call choose the kernel shape (rows
 * per wave, parts a row is cut into, tokens per pass) and with it the order of
 * the fp32 additions over a row's groups.  The same job alone, among 23 others,
 * or at batch 3 instead of 4 may differ in its last bits, always inside the
 * bound; the reference's identities "batch == per token" and "tiles == whole"
 * (tools/test/gemma4-bit-identity-test.c:88-144) hold for the bit-exact
 * kernels only.  For one and the same call the result is reproducible bit
 * for bit, run after run: no atomics, no dependence on workgroup order. */
int salt_mi355_q4_matvec_t_dev(const void *vals, const void *scales, const void *biases,
                               int R, int C, int B, const float *xs, float *ys, void *stream);
int salt_mi355_q4_jobs_t_dev(const SaltMi355Q4Job *jobs, int njobs, int C, int tokens, void *stream);

/* Prefill-sized variant on the matrix cores: ys[t*R + r] for B tokens against
 * one matrix, fp32-accurate but NOT bit-identical to the reference (different
 * summation order): per output
 *   |error| <= 2^-20 * sum_c (|q_c s| + 16 |s| + |b|) |x_c| + 1e-6
 * (and <= 2^-18 * sum_c |w*x| + 1e-6 for activations without outliers).  Needs
 * C % 64 == 0 and device scratch of salt_mi355_q4_matmul_workspace_bytes().
 * The reference has no counterpart: its CPU and GPU paths keep the 32-chain
 * order at every batch size (kernels.c:1252-1261). */
size_t salt_mi355_q4_matmul_workspace_bytes(int C, int B);
int salt_mi355_q4_matmul_dev(const void *vals, const void *scales, const void *biases,
                             int R, int C, int B, const float *xs, float *ys,
                             void *workspace, void *stream);

/* ---- NVFP4, device-resident ---------------------------------------------
 * Layout as the reference's nvfp4.h:37-46: packed E2M1 codes, low nibble =
 * even element; E4M3FN scales [R][C/16]; one fp32 stored divisor per tensor
 * (weight_global_scale = 1 / divisor). */

/* Dynamic group-16 activation quantise/dequantise of B rows of C floats
 * (reference salt_nvfp4_quantize_input_reference, nvfp4.c:82-130).  packed
 * (B*C/2 bytes) and scales (B*C/16 bytes) may be NULL when only the
 * dequantised activation is wanted.  *status_dev (device int, cleared by the
 * caller) is set to -1 when an input is not finite; the reference rejects the
 * call in that case and so must the caller. */
int salt_mi355_nvfp4_qdq_dev(const float *input, int C, int B, float input_global_scale,
                             uint8_t *packed, uint8_t *scales, float *dequant,
                             int *status_dev, void *stream);
/* Rows against an activation that is used as given: pass the dequantised
 * output of salt_mi355_nvfp4_qdq_dev to reproduce the reference matvec
 * (nvfp4.c:228-256), or the raw activation for the weights-only variant. */
int salt_mi355_nvfp4_matvec_dev(const void *packed, const void *scales, float stored_divisor,
                                int R, int C, int B, const float *xs, float *ys,
                                int chains_per_lane, void *stream);

/* Many NVFP4 matrices in one launch (the shape of reference
 * salt_gpu_nvfp4_mixed_batch, gpu.h:55-59): job j multiplies its own
 * R_j x C matrix with its own tokens, the activation used as given (pass the
 * dequantised output of salt_mi355_nvfp4_qdq_dev for the reference matvec).
 * `jobs` is a HOST array; the library copies it to the device on `stream`. */
typedef struct SaltMi355Fp4Job {
    const void *packed;
    const void *scales;
    float stored_divisor;
    const float *xs;         /* device, [tokens][C] */
    float *ys;               /* device, [tokens][rows] */
    int rows;
} SaltMi355Fp4Job;
int salt_mi355_nvfp4_jobs_dev(const SaltMi355Fp4Job *jobs, int njobs, int C, int tokens,
                              int chains_per_lane, void *stream);

/* The reference matvec of one token in one launch (reference
 * salt_nvfp4_matvec_reference, nvfp4.c:228-256): every workgroup quantises
 * and dequantises the activation x[C] itself (nvfp4.c:82-130) and computes its
 * rows from that, bit-identical to salt_mi355_nvfp4_qdq_dev followed by
 * salt_mi355_nvfp4_matvec_dev.  C a multiple of 32, at most 8192.  status_dev:
 * a device int the caller has cleared; it becomes -1 when x holds a non-finite
 * value, and y is not written then. */
int salt_mi355_nvfp4_matvec_qdq_dev(const void *packed, const void *scales,
                                    float stored_divisor, float input_global_scale,
                                    int R, int C, const float *x, float *y,
                                    int *status_dev, int chains, void *stream);

/* Tolerance-class reference matvec: the memory-bound kernel.  Every token is
 * quantised as salt_nvfp4_quantize_input_reference does (nvfp4.c:82-130, the
 * same codes and block scales) inside the launch, and ys[token][row]
 * approximates the reference matvec (nvfp4.c:228-256): per 16-column block the
 * sum of code products is exact, the block's two factors are applied once and
 * the blocks are added in fp32 in a different order than the reference's 32
 * chains.  Bound per output: |y - y_ref| <= 2^-20 * sum_c |w_c x_c|.  xs:
 * [B][C] raw fp32 activations, 16-byte aligned; ys: [B][R].  *status_dev (device
 * int, cleared by the caller) becomes -1 when a token of a job holds a
 * non-finite value; that job then publishes nothing.  C a multiple of 64 from
 * 512 to 8192 takes the streaming kernel, other multiples of 32 the bit-exact
 * one-launch kernel.  The reference has no counterpart. */
int salt_mi355_nvfp4_matvec_t_dev(const void *packed, const void *scales,
                                  float stored_divisor, float input_global_scale,
                                  int R, int C, int B, const float *xs, float *ys,
                                  int *status_dev, void *stream);
int salt_mi355_nvfp4_jobs_t_dev(const SaltMi355Fp4Job *jobs, int njobs, int C, int tokens,
                                float input_global_scale, int *status_dev, void *stream);

/* Prefill-sized NVFP4 matmul on the matrix cores (tolerance class): every
 * token is quantised and dequantised as salt_nvfp4_quantize_input_reference
 * does (nvfp4.c:82-130) and ys[token][row] approximates the reference matvec
 * (nvfp4.c:228-256) of that token: code * block scale is exact in bf16 for both
 * operands, products are exact, fp32 accumulation runs in the matrix cores'
 * order and the two per-tensor factors are applied once at the end.
 * xs: [B][C] fp32, ys: [B][R]; C a multiple of 64.  status_dev (optional device
 * int) receives 0 or -1 (a non-finite activation: nothing is published) and
 * the call stays asynchronous; without it the call waits and returns -1. */
size_t salt_mi355_nvfp4_matmul_workspace_bytes(int R, int C, int B);
int salt_mi355_nvfp4_matmul_dev(const void *packed, const void *scales,
                                float stored_divisor, float input_global_scale,
                                int R, int C, int B, const float *xs, float *ys,
                                int *status_dev, void *workspace, void *stream);

/* ---- the formats themselves, device-resident ----------------------------- */

/* reference salt_q4_decode (src/kernels.c:188-208): out[k] for n flat elements,
 * the scale and bias of group k / 64, two roundings per element; any byte
 * alignment of vals / scales / biases, biases may be NULL.  Bit-exact. */
int salt_mi355_q4_decode_dev(const void *vals, const void *scales, const void *biases,
                             size_t n, float *out, void *stream);
/* reference salt_nvfp4_dequantize_weights_reference (src/nvfp4.c:132-155):
 * out[R*C] = e2m1(code) * (e4m3(scale) * (1 / stored_divisor)).  Bit-exact. */
int salt_mi355_nvfp4_dequant_weights_dev(const void *packed, const void *scales,
                                         float stored_divisor, int R, int C,
                                         float *out, void *stream);
/* reference salt_router (src/router.c:22-57), the fixture router: scores are
 * hashes of (state, layer, expert); idx[topk] in selection order, w[topk] the
 * unbiased scores.  n_experts <= 1024.  Bit-exact (indices and weight bits). */
int salt_mi355_router_fixture_dev(int n_experts, int topk, uint64_t state, int layer,
                                  double locality, int *idx, float *w, void *stream);

/* ---- bf16 and 8-bit affine matvecs, device-resident --------------------- */

/* reference salt_bf16_matvec (src/kernels.c:139-174), the arithmetic behind
 * salt_gpu_bf16_matvec (include/salt/gpu.h:63-65, src/gpu_hip.cpp:1308-1341,
 * 4591-4622): the language-model head.  weights is [R][C] bf16, xs [B][C],
 * ys [B][R], bias [R] or NULL.  Eight column chains per row, the reference's
 * fold tree, separately rounded products and sums: bit-exact.  Any C and any
 * weight address are accepted; C % 8 == 0 with 16-byte aligned weights runs
 * the streaming kernel. */
int salt_mi355_bf16_matvec_dev(const void *weights, int R, int C, int B,
                               const float *xs, const float *bias, float *ys,
                               void *stream);

/* reference salt_q8_matvec (src/kernels.c:343-370), the arithmetic behind
 * salt_gpu_q8_matvec / salt_gpu_q8_batch (include/salt/gpu.h:37-39, 89-94):
 * router gates.  vals is [R][C] bytes, scales and biases (or NULL) one bf16
 * per 64 flat elements.  One left-to-right chain per row: bit-exact. */
int salt_mi355_q8_matvec_dev(const void *vals, const void *scales,
                             const void *biases, int R, int C, int B,
                             const float *xs, float *ys, void *stream);

/* ---- fp32 cells of a decoder block, device-resident --------------------- */

/* One cell of salt_gpu_exact_cells (include/salt/gpu.h:211-234) over device
 * pointers.  kind and the meaning of views, n, aux, eps and scalar are the
 * reference's (src/gpu_hip.cpp:5299-5400):
 *   1 RMSNORM            views: x, weight (read when aux = 1), out
 *   2 TOPK               views: logits, per-expert scale, selected (int), weights; n experts, aux = k; ascending ids
 *   3 RESIDUAL_POSTNORM  views: residual, branch, weight, out
 *   4 PARALLEL_COMBINE   views: residual, dense, routed, dense / routed / final post-norm weights, scratch (2n), out
 *   5 SOFTCAP            views: logits (in place); scalar = cap
 *   6 ROUTER_INPUT       views: state, scale, out; scalar = 1/sqrt(n) or 0 to have it computed
 * Arithmetic: gemma4.c:46-130, 188-286 (serial sum of squares, pow(., -0.5)
 * by double Newton steps, separately rounded products): bit-exact. */
typedef struct SaltMi355Cell {
    int kind;
    const void *views[8];
    uint32_t n, aux;
    float eps, scalar;
} SaltMi355Cell;

/* Enqueues the cells in order.  status_dev points at two device ints that the
 * caller has cleared: [0] becomes -1 when a cell meets a non-finite input or
 * result (that cell and every later one then publish nothing), [1] is scratch. */
int salt_mi355_cells_dev(const SaltMi355Cell *cells, int count, int *status_dev,
                         void *stream);

/* The feed-forward half of one decoder layer for one token, reference
 * feed_forward (models/gemma4-26b-a4b/src/gemma4_text.c:8308-8390): pre-norm,
 * dense gate/up (affine Q4), gelu * up, dense down; router input, 8-bit router
 * gate, top-k; second pre-norm, routed experts, weighted sum; parallel
 * combine.  Every pointer is a device pointer; Q4 and 8-bit tensors are
 * {values, scales, biases}. */
typedef struct SaltMi355FfnLayer {
    int hidden, dense, routed, n_experts, topk;
    float eps, layer_scalar;
    const float *pre_norm, *pre_norm_2, *router_scale, *per_expert_scale;
    const float *post_norm_1, *post_norm_2, *post_norm;
    const void *dense_gate[3], *dense_up[3], *dense_down[3];
    const void *router[3];
    const void *pool;          /* expert 0 */
    size_t expert_stride;
} SaltMi355FfnLayer;

size_t salt_mi355_ffn_block_workspace_bytes(const SaltMi355FfnLayer *layer);
/* residual and out hold `hidden` floats (distinct buffers); selected / weights
 * receive the sorted routing (topk entries).  *status_dev (one device int,
 * cleared by the call) becomes -1 when any step rejects its input; out is then
 * not written.  workspace: 256-byte aligned, sized by the query above. */
int salt_mi355_ffn_block_dev(const SaltMi355FfnLayer *layer, const float *residual,
                             float *out, int *selected, float *weights,
                             int *status_dev, void *workspace, void *stream);

/* ---- MoE decode layer-step, device-resident ----------------------------- */

/* reference salt_gemma4_router_topk (gemma4.c:132-186).  sorted_by_id = 0
 * keeps the reference function's descending-logit order, 1 applies its
 * callers' ascending-expert sort (gemma4_text.c:7923-7930).  *status_dev is
 * set to 0, or to -1 when the reference would return -1 (outputs untouched). */
int salt_mi355_router_topk_dev(const float *logits, const float *per_expert_scale,
                               int n_experts, int topk, int sorted_by_id,
                               int *selected, float *weights, int *status_dev, void *stream);

/* One token through one MoE layer: router top-k, ascending sort, the selected
 * experts (gate, up, gelu*up, down; all affine-Q4 group 64) and the in-order
 * weighted sum (reference gemma4_text.c:8360, 7923-7930, 7608-7649,
 * 8301-8304).  pool = expert 0 of the layer in the engine's slot layout
 * [gate|up|down] x [vals|scales|biases] (gemma4_text.c:73-79), experts
 * expert_stride bytes apart.  selected/weights: topk entries; expert_out
 * (optional): [topk][hidden]; out: [hidden].  workspace: device memory of
 * salt_mi355_moe_workspace_bytes(); its first int receives the router status
 * (0 / -1) and must be read after the stream has drained. */
size_t salt_mi355_moe_workspace_bytes(int hidden, int routed, int n_experts, int topk);
int salt_mi355_moe_decode_step_dev(const void *pool, size_t expert_stride,
                                   int hidden, int routed, int n_experts, int topk,
                                   const float *logits, const float *per_expert_scale,
                                   const float *x, int *selected, float *weights,
                                   float *expert_out, float *out,
                                   void *workspace, void *stream);
/* Tolerance-class form of the layer-step: router top-k, selection and weights
 * are bit-identical to the reference; the three projections of every selected
 * expert run on the kernel of salt_mi355_q4_matvec_t_dev (its bound applies to
 * each projection against its own input), gelu_tanh and the ordered weighted
 * sum are the reference's.  Stated tolerance of the composition (tests), per
 * output and relative to the magnitudes of the output's own terms, with
 * h_k = gelu_tanh(gate_k) * up_k and Wd_k the dequantised down projection:
 *   |expert_out[k][d] - ref| <= 2^-18 * sum_f |Wd_k[d][f] * h_k[f]| + 1e-6,
 *   |out[d] - ref| <= 2^-18 * sum_k |w_k| * sum_f |Wd_k[d][f] * h_k[f]| + 1e-6.
 * Same arguments and workspace as salt_mi355_moe_decode_step_dev; more than
 * 256 experts or widths the streaming kernels do not take (fewer than 512
 * columns, more than 8192) run the bit-exact plan.  As for every
 * tolerance-class entry point the bits depend on the launch (here: on the
 * geometry), not on the run. */
int salt_mi355_moe_decode_step_t_dev(const void *pool, size_t expert_stride,
                                     int hidden, int routed, int n_experts, int topk,
                                     const float *logits, const float *per_expert_scale,
                                     const float *x, int *selected, float *weights,
                                     float *expert_out, float *out,
                                     void *workspace, void *stream);
/* The same layer-step for callers that cannot allocate device memory or pass a
 * workspace (code under HIP graph capture, tight serving loops, harnesses that
 * forbid hipMalloc): the workspace is a static array inside the library, one
 * per device, SALT_MI355_MOE_STATIC_SCRATCH_BYTES large, and the call allocates
 * nothing.  It has no counterpart in the reference.  Geometries whose
 * salt_mi355_moe_workspace_bytes() exceeds the array are refused (-1).  Results
 * are bit-identical to salt_mi355_moe_decode_step_dev.  status_dev (optional
 * device int) receives the router status (0 / -1).  All calls on one device
 * share the array: calls that overlap in time on one device (two streams) race. */
#define SALT_MI355_MOE_STATIC_SCRATCH_BYTES (1 << 20)
int salt_mi355_moe_decode_step_static_dev(const void *pool, size_t expert_stride,
                                          int hidden, int routed, int n_experts, int topk,
                                          const float *logits, const float *per_expert_scale,
                                          const float *x, int *selected, float *weights,
                                          float *expert_out, float *out,
                                          int *status_dev, void *stream);
/* Many tokens through the experts of one MoE layer, grouped per expert
 * (reference src/moe_group.c:24-97 validation, :138-184 grouping in ascending
 * expert / token / rank order, :211-224 weighted sum over ranks in rank order
 * from +0; per-expert arithmetic gemma4_text.c:8749-9137).  The bucketing is
 * exact; the projections run on the matrix-core kernel of
 * salt_mi355_q4_matmul_dev and carry its tolerance.  selected / weights:
 * [tokens][topk] (any order inside a token; experts distinct, weights
 * finite); inputs / outputs: [tokens][hidden].  Optional results: group_rows
 * [n_experts] rows per expert, row_pairs [tokens*topk] the pair index
 * token*topk+rank of each grouped row.  status_dev (optional device int):
 * receives 0 or -1 and the call stays asynchronous; without it the call waits
 * for the stream and returns -1 for an invalid selection.  Outputs are not
 * written for an invalid selection. */
size_t salt_mi355_moe_prefill_workspace_bytes(int hidden, int routed, int n_experts, int topk, int tokens);
int salt_mi355_moe_prefill_dev(const void *pool, size_t expert_stride,
                               int hidden, int routed, int n_experts, int topk, int tokens,
                               const int *selected, const float *weights,
                               const float *inputs, float *outputs,
                               int *group_rows, int *row_pairs, int *status_dev,
                               void *workspace, void *stream);
/* The pieces of the step on their own: act = gelu_tanh(gate) * up over n
 * floats (gemma4.c:80-83, gemma4_text.c:7635), and out[d] = sum_i
 * expert_out[i][d] * weights[i] from +0 in ascending i (gemma4_text.c:8301-8304). */
int salt_mi355_moe_activate_dev(const float *gate, const float *up, float *act, size_t n, void *stream);
int salt_mi355_moe_reduce_dev(const float *expert_out, const float *weights, int topk, int hidden,
                              float *out, void *stream);

#ifdef __cplusplus
}
#endif

#endif /* SALT_GPU_MI355_H */
