/* salt_oracle.h -- CPU restatement of SALT's quantized decode arithmetic.
 *
 * TEST INFRASTRUCTURE ONLY.  Nothing in the shipped library links, loads or
 * calls this code: it exists so that the parity tests, the smoke check and
 * the CPU-baseline leg of the benchmark have an independent statement of the
 * reference algorithm to compare the HIP kernels against.
 *
 * Every function names the reference lines it restates.  All arithmetic is
 * IEEE binary32 with one rounding per operator; build with
 * -ffp-contract=off (the Makefile next to this file does).
 */
#ifndef SALT_ORACLE_H
#define SALT_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- affine Q4 ("mlx4"): u32 words of 8 nibbles, bf16 scale+bias per 64 */

/* reference src/kernels.c:118-123 */
float orc_bf16(uint16_t half);
/* reference src/kernels.c:188-208 (salt_q4_decode) */
void orc_q4_decode(const void *vals, const void *scales, const void *biases,
                   size_t n, float *out);
/* reference src/kernels.c:220-250 (q4_canonical_row) */
float orc_q4_row(const void *vals, const void *scales, const void *biases,
                 int C, const float *x, int row);
/* reference src/kernels.c:252-274, 283-335 (validation + row loop) */
int orc_q4_matvec(const void *vals, const void *scales, const void *biases,
                  int R, int C, const float *x, float *y);
int orc_q4_matvec_rows(const void *vals, const void *scales,
                       const void *biases, int R, int C, const float *x,
                       float *y, int r0, int r1);
/* reference src/kernels.c:1252-1306: ys[t*R+r] = row r against xs[t*C..] */
int orc_q4_matvec_batch(const void *vals, const void *scales,
                        const void *biases, int R, int C, int B,
                        const float *xs, float *ys);
/* Row-split over `threads` pthreads by the reference's rule
 * (chunk = ceil(R/threads), src/kernels.c:291-323).  Same bits as the
 * single-thread call; used for the timed CPU baseline. */
int orc_q4_matvec_threads(const void *vals, const void *scales,
                          const void *biases, int R, int C, const float *x,
                          float *y, int threads);

/* ---- bf16 and 8-bit affine matvecs (the LM head and the router gates) */

/* reference src/kernels.c:139-174 (salt_bf16_matvec, scalar body): eight
 * chains a[c % 8] over the 8-aligned part of the row, each p = fl(w*x),
 * a = fl(a + p); s = ((a0+a2)+(a4+a6)) + ((a1+a3)+(a5+a7)); the columns past
 * the last multiple of eight are added to s in order; y = s + (bias ? bias[r]
 * : 0.0f). */
void orc_bf16_matvec(const uint16_t *W, int R, int C, const float *x,
                     const float *bias, float *y);
/* reference src/kernels.c:343-370 (salt_q8_matvec): one chain per row,
 * acc = fl(acc + fl(fl(fl(q*s) + b) * x[c])) over all columns in order; the
 * value of flat element k is byte k of vals, its scale group k / 64. */
void orc_q8_matvec(const void *vals, const void *scales, const void *biases,
                   int R, int C, const float *x, float *y);

/* ---- NVFP4: packed E2M1 codes, E4M3FN block scale per 16, fp32 divisor */

/* reference src/nvfp4.c:19-23 */
float orc_e2m1(uint8_t code);
/* reference src/nvfp4.c:25-39 */
float orc_e4m3fn(uint8_t code);
/* reference src/nvfp4.c:41-63 (argmin scan, ties to even code) */
int orc_e4m3fn_encode(float value, uint8_t *code);
/* reference src/nvfp4.c:65-80 */
uint8_t orc_e2m1_encode(float value);
/* Closed-form round-to-nearest-even encoders; the HIP kernels use the same
 * closed forms, and the tests prove them equal to the scans above. */
uint8_t orc_e4m3fn_encode_rne(float value);
uint8_t orc_e2m1_encode_rne(float value);
/* reference src/nvfp4.c:82-130 */
int orc_nvfp4_qdq(const float *input, int C, float input_global_scale,
                  uint8_t *packed, uint8_t *scales, float *dequant);
/* reference src/nvfp4.c:132-155 */
int orc_nvfp4_dequant_weights(const uint8_t *packed, const uint8_t *scales,
                              float stored_divisor, int R, int C, float *out);
/* reference src/nvfp4.c:157-192 (row with a given dequantised activation) */
float orc_nvfp4_row(const uint8_t *packed, const uint8_t *scales,
                    float weight_global_scale, int row, int C,
                    const float *x_dq);
/* reference src/nvfp4.c:228-256 */
int orc_nvfp4_matvec(const uint8_t *packed, const uint8_t *scales,
                     float stored_divisor, float input_global_scale,
                     int R, int C, const float *input, float *output,
                     uint8_t *x_packed, uint8_t *x_scales, float *x_dq);
/* Rows against an activation that is used as given (no Q/DQ pre-pass). */
int orc_nvfp4_matvec_weights_only(const uint8_t *packed,
                                  const uint8_t *scales, float stored_divisor,
                                  int R, int C, const float *x, float *output);

/* ---- deterministic transcendentals */

/* reference src/bitmath.c:44-63 */
float orc_expf(float x);
/* reference src/bitmath.c:144-153 */
float orc_tanhf(float x);
/* reference models/gemma4-26b-a4b/src/gemma4.c:80-83 */
float orc_gelu_tanh(float x);

/* reference src/bitmath.c:117-142 (six double Newton steps from the
 * 0x5f3759df seed; tiny inputs rescaled by 2^24) */
float orc_rsqrtf(float x);
float orc_sqrtf(float x);
/* reference src/bitmath.c:107-112 restricted to the exponent -0.5, the only
 * one the norms use */
float orc_pow_minus_half(float x);

/* ---- norms and residual combinations of the decoder block (all reject
 *      non-finite inputs or results with -1 and then write nothing) */

/* reference gemma4.c:46-71, 85-101: ss = serial sum of x*x; inv =
 * pow(ss / n + eps, -0.5); out = (x * inv) * weight (weight only when
 * with_scale) */
int orc_rmsnorm(float *out, const float *x, const float *weight, int n,
                float eps, int with_scale);
/* reference gemma4.c:103-130: ((state * inv) * scale) * (1 / sqrt(hidden)) */
int orc_router_input(float *out, const float *state, const float *scale,
                     int hidden, float eps);
/* reference gemma4.c:188-214: residual + (branch * inv) * weight */
int orc_residual_postnorm(float *out, const float *residual,
                          const float *branch, const float *weight, int n,
                          float eps);
/* reference gemma4.c:216-276: norm(dense) + norm(routed), norm of that sum,
 * (residual + it) * layer_scalar */
int orc_parallel_ffn_combine(float *out, const float *residual,
                             const float *dense, const float *routed,
                             const float *dense_post_weight,
                             const float *routed_post_weight,
                             const float *final_post_weight,
                             float layer_scalar, int n, float eps);
/* reference gemma4.c:278-286: cap * tanh(logit / cap), in place */
int orc_softcap(float *logits, int n, float cap);

/* ---- routers */

/* reference models/gemma4-26b-a4b/src/gemma4.c:132-186 */
int orc_router_topk(const float *logits, const float *per_expert_scale,
                    int n_experts, int topk, int *selected, float *weights);
/* reference models/gemma4-26b-a4b/src/gemma4_text.c:7923-7930 */
void orc_sort_selection(int *selected, float *weights, int topk);
/* reference src/router.c:11-20 */
uint64_t orc_mix64(uint64_t x);
/* reference src/router.c:22-57 (fixture router) */
int orc_router_fixture(int *idx, float *w, int n_experts, int topk,
                       uint64_t state, int layer, double locality);

/* ---- routed expert FFN and MoE layer */

/* Byte geometry of one expert in the pool: [gate|up|down], each projection
 * [vals|scales|biases] (reference gemma4_text.c:73-79, 7608-7612). */
typedef struct OrcExpertGeometry {
    int hidden;      /* d_model, columns of gate/up, rows of down   */
    int routed;      /* d_ff, rows of gate/up, columns of down      */
} OrcExpertGeometry;
size_t orc_expert_proj_bytes(const OrcExpertGeometry *g);
size_t orc_expert_slot_bytes(const OrcExpertGeometry *g);

/* reference gemma4_text.c:7608-7649 (expert_worker): gate, up, gelu*up,
 * down.  gate/up scratch hold `routed` floats, output `hidden` floats. */
int orc_expert_ffn(const OrcExpertGeometry *g, const unsigned char *slot,
                   const float *input, float *gate, float *up, float *output);
/* One decode layer-step: router top-k, ascending sort, the selected
 * experts, and the in-order weighted sum (reference gemma4_text.c:8360,
 * 7923-7930, 7608-7649, 8301-8304).  pool points at expert 0 of the layer;
 * experts are orc_expert_slot_bytes apart.  expert_out (optional) receives
 * the topk per-expert outputs [topk][hidden] in sorted order. */
int orc_moe_decode_step(const OrcExpertGeometry *g, const unsigned char *pool,
                        int n_experts, int topk, const float *logits,
                        const float *per_expert_scale, const float *input,
                        int *selected, float *weights, float *expert_out,
                        float *output, int threads);
/* Grouped prefill MoE: validation, ascending-expert / token / rank row
 * order, per-expert batch FFN, scatter to [token][rank] slots, in-order
 * weighted reduce (reference src/moe_group.c:83-97, 138-224 with the Gemma
 * group ops gemma4_text.c:8749-9137 doing gate/up -> gelu*up -> down).
 * group_rows (optional, n_experts ints) receives each expert's row count. */
int orc_moe_group(const OrcExpertGeometry *g, const unsigned char *pool,
                  int n_experts, int topk, int batch, const int *selected,
                  const float *weights, const float *inputs, float *outputs,
                  int *group_rows, int threads);

/* ---- the feed-forward half of one decoder layer, one token */

/* Weights of one layer's feed-forward block.  Q4 tensors are [vals|scales|
 * biases] pointer triples; the router gate is 8-bit affine. */
typedef struct OrcFfnLayer {
    int hidden, dense, routed, n_experts, topk;
    float eps, layer_scalar;
    const float *pre_norm, *pre_norm_2, *router_scale, *per_expert_scale;
    const float *post_norm_1, *post_norm_2, *post_norm;
    const void *dense_gate[3], *dense_up[3], *dense_down[3];
    const void *router[3];
    const unsigned char *pool;       /* expert 0; orc_expert_slot_bytes apart */
} OrcFfnLayer;

/* reference gemma4_text.c:8308-8390 (feed_forward): pre-norm, dense gate/up,
 * gelu * up, dense down; router input, 8-bit gate, top-k, ascending sort;
 * second pre-norm, routed experts, weighted sum; parallel combine.
 * selected / weights (optional) receive the sorted routing. */
int orc_ffn_block(const OrcFfnLayer *layer, const float *residual,
                  float *output, int *selected, float *weights, int threads);

#ifdef __cplusplus
}
#endif

#endif /* SALT_ORACLE_H */
