/* salt_oracle.c -- CPU restatement of SALT's quantized decode arithmetic.
 *
 * TEST INFRASTRUCTURE ONLY (see salt_oracle.h).  Each function cites the
 * reference lines whose behaviour it restates.  One IEEE binary32 rounding
 * per operator, no fused multiply-add: build with -ffp-contract=off.
 *
 * What pins each function (tests/test_oracle_*.py):
 *   orc_q4_decode / orc_q4_row / orc_q4_matvec*  reference known answers
 *       (tests/test_kernels.c:357-392, 453-521), a step-by-step numpy
 *       float32 emulation, exact power-of-two scaling, row independence,
 *       the compiled reference (oracle/_ref) and fixtures made from it.
 *   orc_e2m1 / orc_e4m3fn / encoders / orc_nvfp4_qdq / orc_nvfp4_matvec
 *       reference golden bytes and bit patterns (tests/test_nvfp4.c:28-117),
 *       OCP FP8/FP4 tables from torch, the compiled reference and fixtures.
 *   orc_bf16_matvec / orc_q8_matvec   the compiled reference in both its
 *       scalar and SIMD realisation, a step-by-step numpy float32
 *       emulation, exact closed forms (powers of two against the column
 *       index; byte sums; a single left-to-right chain).
 *   orc_expf / orc_tanhf / orc_gelu_tanh   no vectors exist in the reference
 *       tree; pinned by fixtures generated from the compiled reference and by
 *       closeness to libm (a dropped Horner term or a wrong constant fails).
 *   orc_rsqrtf / orc_sqrtf / orc_pow_minus_half   exact powers of four, libm
 *       within one ulp, the compiled reference on 20k points and the edges.
 *   orc_rmsnorm / orc_router_input / orc_residual_postnorm /
 *   orc_parallel_ffn_combine / orc_softcap   the compiled reference
 *       (bit-equal outputs, same rejections), closed forms (constant
 *       vectors, a 2^24 + 1 + 1 ... chain that a tree would round
 *       differently, cancelling branches).
 *   orc_ffn_block   the compiled reference's public constituents driven in
 *       feed_forward's order (feed_forward is a static function of the model
 *       file).
 *   orc_router_topk / orc_sort_selection   brute-force ordering on small E,
 *       weight identities, fixtures from the compiled reference.
 *   orc_mix64 / orc_router_fixture         splitmix64 published test values,
 *       brute-force top-k, fixtures from the compiled reference.
 *   orc_expert_ffn / orc_moe_decode_step / orc_moe_group   composition of the
 *       above; closed forms with identity-like experts; fixtures from the
 *       compiled reference (expert_worker itself is a static function of
 *       gemma4_text.c, so the fixture drives its public constituents in the
 *       same order).
 */
#include "salt_oracle.h"

#include <float.h>
#include <math.h>
#include <pthread.h>
#include <stdlib.h>
#include <string.h>

#define ORC_GROUP 64u

/* ------------------------------------------------------------------ */
/* byte-addressed loads: sources may sit on any byte boundary          */
/* (reference src/kernels.c:125-137, tests/test_kernels.c:480-521)     */
/* ------------------------------------------------------------------ */

static uint32_t ld32(const void *base, size_t index) {
    uint32_t v;
    memcpy(&v, (const unsigned char *)base + 4u * index, 4);
    return v;
}

static uint16_t ld16(const void *base, size_t index) {
    uint16_t v;
    memcpy(&v, (const unsigned char *)base + 2u * index, 2);
    return v;
}

float orc_bf16(uint16_t half) {
    uint32_t wide = (uint32_t)half << 16;
    float f;
    memcpy(&f, &wide, 4);
    return f;
}

static unsigned q4_nibble(const void *vals, size_t k) {
    return (ld32(vals, k >> 3) >> (4u * (unsigned)(k & 7u))) & 15u;
}

/* ------------------------------------------------------------------ */
/* affine Q4                                                           */
/* ------------------------------------------------------------------ */

void orc_q4_decode(const void *vals, const void *scales, const void *biases,
                   size_t n, float *out) {
    for (size_t k = 0; k < n; k++) {
        size_t g = k / ORC_GROUP;
        float s = orc_bf16(ld16(scales, g));
        float b = biases ? orc_bf16(ld16(biases, g)) : 0.0f;
        float scaled = (float)q4_nibble(vals, k) * s;
        out[k] = scaled + b;
    }
}

/* The fold shared by Q4 and NVFP4 rows: four partial sums over the 32
 * accumulators taken with stride 4 starting from +0, then
 * (p0 + p2) + (p1 + p3).  reference src/kernels.c:239-249,
 * src/nvfp4.c:157-171. */
static float fold32(const float acc[32]) {
    float part[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    for (int a = 0; a < 8; a++)
        for (int j = 0; j < 4; j++)
            part[j] = part[j] + acc[4 * a + j];
    float even = part[0] + part[2];
    float odd = part[1] + part[3];
    return even + odd;
}

float orc_q4_row(const void *vals, const void *scales, const void *biases,
                 int C, const float *x, int row) {
    float acc[32];
    size_t first = (size_t)row * (size_t)C;
    for (int j = 0; j < 32; j++) acc[j] = 0.0f;
    for (int c = 0; c < C; c++) {
        size_t k = first + (size_t)c;
        size_t g = k / ORC_GROUP;
        float s = orc_bf16(ld16(scales, g));
        float b = biases ? orc_bf16(ld16(biases, g)) : 0.0f;
        float w = (float)q4_nibble(vals, k) * s;
        w = w + b;
        float p = w * x[c];
        acc[c & 31] = acc[c & 31] + p;
    }
    return fold32(acc);
}

int orc_q4_matvec_rows(const void *vals, const void *scales,
                       const void *biases, int R, int C, const float *x,
                       float *y, int r0, int r1) {
    if (!vals || !scales || !x || !y || R < 1 || C < 1 || r0 < 0 ||
        r1 < r0 || r1 > R || (size_t)R > SIZE_MAX / (size_t)C)
        return -1;
    for (int r = r0; r < r1; r++)
        y[r] = orc_q4_row(vals, scales, biases, C, x, r);
    return 0;
}

int orc_q4_matvec(const void *vals, const void *scales, const void *biases,
                  int R, int C, const float *x, float *y) {
    return orc_q4_matvec_rows(vals, scales, biases, R, C, x, y, 0, R);
}

int orc_q4_matvec_batch(const void *vals, const void *scales,
                        const void *biases, int R, int C, int B,
                        const float *xs, float *ys) {
    if (B < 1 || !xs || !ys) return -1;
    for (int t = 0; t < B; t++)
        if (orc_q4_matvec(vals, scales, biases, R, C,
                          xs + (size_t)t * (size_t)C,
                          ys + (size_t)t * (size_t)R) != 0)
            return -1;
    return 0;
}

typedef struct {
    const void *vals, *scales, *biases;
    int R, C, r0, r1;
    const float *x;
    float *y;
} Q4Span;

static void *q4_span_main(void *opaque) {
    Q4Span *s = (Q4Span *)opaque;
    for (int r = s->r0; r < s->r1; r++)
        s->y[r] = orc_q4_row(s->vals, s->scales, s->biases, s->C, s->x, r);
    return NULL;
}

int orc_q4_matvec_threads(const void *vals, const void *scales,
                          const void *biases, int R, int C, const float *x,
                          float *y, int threads) {
    pthread_t tid[64];
    Q4Span span[64];
    int live[64];
    if (!vals || !scales || !x || !y || R < 1 || C < 1) return -1;
    if (threads < 1) threads = 1;
    if (threads > 64) threads = 64;
    int chunk = R / threads + (R % threads != 0);
    for (int t = 0; t < threads; t++) {
        long long a = (long long)t * chunk, b = a + chunk;
        Q4Span *s = &span[t];
        s->vals = vals; s->scales = scales; s->biases = biases;
        s->R = R; s->C = C; s->x = x; s->y = y;
        s->r0 = a < R ? (int)a : R;
        s->r1 = b < R ? (int)b : R;
        live[t] = 0;
        if (s->r0 >= s->r1) continue;
        if (threads > 1 && pthread_create(&tid[t], NULL, q4_span_main, s) == 0)
            live[t] = 1;
        else
            q4_span_main(s);
    }
    for (int t = 0; t < threads; t++)
        if (live[t]) pthread_join(tid[t], NULL);
    return 0;
}

/* ------------------------------------------------------------------ */
/* NVFP4                                                               */
/* ------------------------------------------------------------------ */

static const float e2m1_magnitude[8] = {0.0f, 0.5f, 1.0f, 1.5f,
                                        2.0f, 3.0f, 4.0f, 6.0f};

float orc_e2m1(uint8_t code) {
    float m = e2m1_magnitude[code & 7u];
    if (m == 0.0f) return 0.0f;            /* "-0" decodes to +0 */
    return (code & 8u) ? -m : m;
}

float orc_e4m3fn(uint8_t code) {
    int e = (code >> 3) & 15, m = code & 7;
    float v;
    if (e == 15 && m == 7) return NAN;
    if (e == 0)
        v = (float)m * 0.001953125f;
    else
        v = (1.0f + (float)m * 0.125f) * ldexpf(1.0f, e - 7);
    return (code & 0x80u) ? -v : v;
}

/* Argmin over the ascending candidate list; on an exact tie the even code
 * replaces an odd incumbent. */
int orc_e4m3fn_encode(float value, uint8_t *code) {
    if (!code || isnan(value)) return -1;
    float m = fabsf(value);
    if (m > 448.0f) m = 448.0f;
    unsigned keep = 0;
    float keep_d = FLT_MAX;
    for (unsigned c = 0; c <= 0x7eu; c++) {
        float d = fabsf(m - orc_e4m3fn((uint8_t)c));
        int closer = d < keep_d;
        int tie_to_even = d == keep_d && !(c & 1u) && (keep & 1u);
        if (closer || tie_to_even) { keep = c; keep_d = d; }
    }
    *code = (uint8_t)(keep | (signbit(value) ? 0x80u : 0u));
    return 0;
}

uint8_t orc_e2m1_encode(float value) {
    float m = fabsf(value);
    unsigned keep = 0;
    float keep_d = FLT_MAX;
    for (unsigned c = 0; c < 8u; c++) {
        float d = fabsf(m - e2m1_magnitude[c]);
        int closer = d < keep_d;
        int tie_to_even = d == keep_d && !(c & 1u) && (keep & 1u);
        if (closer || tie_to_even) { keep = c; keep_d = d; }
    }
    return (uint8_t)(keep | (signbit(value) ? 8u : 0u));
}

/* Closed form of orc_e4m3fn_encode for non-NaN input: below 2^-6 the grid
 * is uniform with step 2^-9, above it the binary32 significand is rounded
 * to three fraction bits, both round-half-even, saturating at 448. */
uint8_t orc_e4m3fn_encode_rne(float value) {
    float m = fabsf(value);
    unsigned sign = signbit(value) ? 0x80u : 0u;
    unsigned code;
    if (m > 448.0f) m = 448.0f;
    if (m < 0.015625f) {
        code = (unsigned)rintf(m * 512.0f);
    } else {
        uint32_t bits;
        memcpy(&bits, &m, 4);
        bits += 0x7FFFFu + ((bits >> 20) & 1u);
        code = (bits >> 20) - ((127u - 7u) << 3);
    }
    return (uint8_t)(code | sign);
}

/* Closed form of orc_e2m1_encode: count the decision thresholds passed;
 * a threshold is inclusive exactly when the code above it is even. */
uint8_t orc_e2m1_encode_rne(float value) {
    float m = fabsf(value);
    unsigned code = (unsigned)(m > 0.25f) + (unsigned)(m >= 0.75f) +
                    (unsigned)(m > 1.25f) + (unsigned)(m >= 1.75f) +
                    (unsigned)(m > 2.5f) + (unsigned)(m >= 3.5f) +
                    (unsigned)(m > 5.0f);
    return (uint8_t)(code | (signbit(value) ? 8u : 0u));
}

int orc_nvfp4_qdq(const float *input, int C, float g, uint8_t *packed,
                  uint8_t *scales, float *dequant) {
    if (!input || !packed || !scales || !dequant || C < 16 || (C & 15) ||
        !isfinite(g) || g <= 0.0f)
        return -1;
    for (int blk = 0; blk < C / 16; blk++) {
        const float *src = input + 16 * blk;
        float top = 0.0f;
        for (int i = 0; i < 16; i++) {
            float m = fabsf(src[i]);
            if (!isfinite(m)) return -1;
            if (m > top) top = m;
        }
        float sixth = top * (1.0f / 6.0f);
        float raw = g * sixth;
        if (raw > 448.0f) raw = 448.0f;
        uint8_t scale_code;
        if (orc_e4m3fn_encode(raw, &scale_code) != 0) return -1;
        scales[blk] = scale_code;
        float scale = orc_e4m3fn(scale_code);
        float to_code = scale == 0.0f ? 0.0f : g / scale;
        float from_code = scale / g;
        for (int i = 0; i < 16; i += 2) {
            uint8_t pair[2];
            for (int h = 0; h < 2; h++) {
                float v = src[i + h] * to_code;
                if (v > 6.0f) v = 6.0f;
                if (v < -6.0f) v = -6.0f;
                pair[h] = orc_e2m1_encode(v);
                dequant[16 * blk + i + h] = orc_e2m1(pair[h]) * from_code;
            }
            packed[(16 * blk + i) / 2] =
                (uint8_t)(pair[0] | (uint8_t)(pair[1] << 4));
        }
    }
    return 0;
}

static unsigned fp4_code(const uint8_t *packed, size_t index) {
    unsigned byte = packed[index >> 1];
    return (index & 1u) ? (byte >> 4) : (byte & 15u);
}

int orc_nvfp4_dequant_weights(const uint8_t *packed, const uint8_t *scales,
                              float stored_divisor, int R, int C, float *out) {
    if (!packed || !scales || !out || R < 1 || C < 16 || (C & 15) ||
        !isfinite(stored_divisor) || stored_divisor == 0.0f)
        return -1;
    float wg = 1.0f / stored_divisor;
    for (int r = 0; r < R; r++)
        for (int c = 0; c < C; c++) {
            size_t k = (size_t)r * (size_t)C + (size_t)c;
            float s = orc_e4m3fn(scales[(size_t)r * (size_t)(C / 16) +
                                        (size_t)(c / 16)]);
            float scaled = s * wg;
            out[k] = orc_e2m1((uint8_t)fp4_code(packed, k)) * scaled;
        }
    return 0;
}

float orc_nvfp4_row(const uint8_t *packed, const uint8_t *scales, float wg,
                    int row, int C, const float *x_dq) {
    float acc[32];
    for (int j = 0; j < 32; j++) acc[j] = 0.0f;
    for (int c = 0; c < C; c++) {
        size_t k = (size_t)row * (size_t)C + (size_t)c;
        float s = orc_e4m3fn(scales[(size_t)row * (size_t)(C / 16) +
                                    (size_t)(c / 16)]);
        float scaled = s * wg;
        float w = orc_e2m1((uint8_t)fp4_code(packed, k)) * scaled;
        float p = w * x_dq[c];
        acc[c & 31] = acc[c & 31] + p;
    }
    return fold32(acc);
}

int orc_nvfp4_matvec(const uint8_t *packed, const uint8_t *scales,
                     float stored_divisor, float input_global_scale,
                     int R, int C, const float *input, float *output,
                     uint8_t *x_packed, uint8_t *x_scales, float *x_dq) {
    if (!packed || !scales || !input || !output || !x_packed || !x_scales ||
        !x_dq || R < 1 || C < 16 || (C & 15) ||
        !isfinite(stored_divisor) || stored_divisor == 0.0f)
        return -1;
    float wg = 1.0f / stored_divisor;
    if (orc_nvfp4_qdq(input, C, input_global_scale, x_packed, x_scales,
                      x_dq) != 0)
        return -1;
    for (int r = 0; r < R; r++)
        output[r] = orc_nvfp4_row(packed, scales, wg, r, C, x_dq);
    return 0;
}

int orc_nvfp4_matvec_weights_only(const uint8_t *packed,
                                  const uint8_t *scales, float stored_divisor,
                                  int R, int C, const float *x, float *output) {
    if (!packed || !scales || !x || !output || R < 1 || C < 16 || (C & 15) ||
        !isfinite(stored_divisor) || stored_divisor == 0.0f)
        return -1;
    float wg = 1.0f / stored_divisor;
    for (int r = 0; r < R; r++)
        output[r] = orc_nvfp4_row(packed, scales, wg, r, C, x);
    return 0;
}

/* ------------------------------------------------------------------ */
/* bf16 and 8-bit affine matvecs                                       */
/* ------------------------------------------------------------------ */

void orc_bf16_matvec(const uint16_t *W, int R, int C, const float *x,
                     const float *bias, float *y) {
    for (int r = 0; r < R; r++) {
        const uint16_t *row = W + (size_t)r * (size_t)C;
        float a[8];
        for (int j = 0; j < 8; j++) a[j] = 0.0f;
        int c = 0;
        for (; c + 7 < C; c += 8)
            for (int j = 0; j < 8; j++) {
                float p = orc_bf16(row[c + j]) * x[c + j];
                a[j] = a[j] + p;
            }
        float even = (a[0] + a[2]) + (a[4] + a[6]);
        float odd = (a[1] + a[3]) + (a[5] + a[7]);
        float s = even + odd;
        for (; c < C; c++) {
            float p = orc_bf16(row[c]) * x[c];
            s = s + p;
        }
        y[r] = s + (bias ? bias[r] : 0.0f);
    }
}

void orc_q8_matvec(const void *vals, const void *scales, const void *biases,
                   int R, int C, const float *x, float *y) {
    const unsigned char *bytes = (const unsigned char *)vals;
    for (int r = 0; r < R; r++) {
        float acc = 0.0f;
        for (int c = 0; c < C; c++) {
            size_t k = (size_t)r * (size_t)C + (size_t)c;
            size_t g = k / ORC_GROUP;
            float s = orc_bf16(ld16(scales, g));
            float b = biases ? orc_bf16(ld16(biases, g)) : 0.0f;
            float w = (float)bytes[k] * s;
            w = w + b;
            float p = w * x[c];
            acc = acc + p;
        }
        y[r] = acc;
    }
}

/* ------------------------------------------------------------------ */
/* deterministic transcendentals                                       */
/* ------------------------------------------------------------------ */

float orc_expf(float x) {
    /* Taylor coefficients 1/8! .. 1/2! as written in the reference. */
    static const float coef[7] = {
        2.48015873015873e-05f, 1.98412698412698e-04f, 1.38888888888889e-03f,
        8.33333333333333e-03f, 4.16666666666667e-02f, 1.66666666666667e-01f,
        5.0e-01f};
    if (x != x) return x;
    if (x > 88.722839f) return 3.402823466e+38f;
    if (x < -87.336548f) return 0.0f;
    double n = round((double)x *
        1.442695040888963407359924681001892137426645954152985934135449406931);
    double r = (double)x - n *
        0.693147180559945309417232121458176568075500134360255254120680009;
    float rf = (float)r;
    float p = coef[0];
    for (int i = 1; i < 7; i++) {
        p = p * rf;
        p = p + coef[i];
    }
    p = p * rf;
    p = p + 1.0f;
    p = p * rf;
    p = p + 1.0f;
    return ldexpf(p, (int)n);
}

float orc_tanhf(float x) {
    if (x != x) return x;
    if (x >= 10.0f) return 1.0f;
    if (x <= -10.0f) return -1.0f;
    float m = x < 0.0f ? -x : x;
    float e = orc_expf(2.0f * m);
    float t = (e - 1.0f) / (e + 1.0f);
    return x < 0.0f ? -t : t;
}

float orc_gelu_tanh(float x) {
    const float k = 0.7978845608028654f;
    float cube = 0.044715f * x;
    cube = cube * x;
    cube = cube * x;
    float inner = x + cube;
    float t = orc_tanhf(k * inner);
    float half = 0.5f * x;
    return half * (1.0f + t);
}

static double inverse_root64(float x) {
    uint32_t bits;
    float seed;
    memcpy(&bits, &x, 4);
    bits = UINT32_C(0x5f3759df) - (bits >> 1);
    memcpy(&seed, &bits, 4);
    double y = (double)seed, wide = (double)x;
    for (int i = 0; i < 6; i++) {
        double square = y * y;
        double half = 0.5 * wide;
        double step = 1.5 - half * square;
        y = y * step;
    }
    return y;
}

float orc_rsqrtf(float x) {
    if (x != x) return x;
    if (x < 0.0f) return NAN;
    if (x == 0.0f) return INFINITY;
    if (x == 1.0f) return 1.0f;
    if (x < 0x1p-126f) return orc_rsqrtf(x * 0x1p24f) * 0x1p12f;
    return (float)inverse_root64(x);
}

float orc_sqrtf(float x) {
    if (x != x) return x;
    if (x < 0.0f) return NAN;
    if (x == 0.0f || x == 1.0f) return x;
    if (x < 0x1p-126f) return orc_sqrtf(x * 0x1p24f) * 0x1p-12f;
    return (float)((double)x * inverse_root64(x));
}

float orc_pow_minus_half(float x) {
    if (x == 1.0f) return 1.0f;
    if (x > 0.0f) return orc_rsqrtf(x);
    return x;
}

/* ------------------------------------------------------------------ */
/* norms and residual combinations                                     */
/* ------------------------------------------------------------------ */

static int ranges_touch(const void *a, size_t na, const void *b, size_t nb);

static int norm_inverse(const float *x, const float *weight, int n, float eps,
                        int with_scale, float *inv_out) {
    float ss = 0.0f;
    if (!x || n < 1 || !(eps >= 0.0f) || !isfinite(eps) ||
        (with_scale && !weight))
        return -1;
    for (int i = 0; i < n; i++) {
        if (!isfinite(x[i]) || (with_scale && !isfinite(weight[i]))) return -1;
        float sq = x[i] * x[i];
        ss = ss + sq;
    }
    float mean = ss / (float)n;
    float inv = orc_pow_minus_half(mean + eps);
    if (!isfinite(inv)) return -1;
    for (int i = 0; i < n; i++) {
        float y = x[i] * inv;
        if (with_scale) y = y * weight[i];
        if (!isfinite(y)) return -1;
    }
    *inv_out = inv;
    return 0;
}

int orc_rmsnorm(float *out, const float *x, const float *weight, int n,
                float eps, int with_scale) {
    float inv;
    if (!out || n < 1) return -1;
    size_t bytes = (size_t)n * 4;
    if ((out != x && x && ranges_touch(out, bytes, x, bytes)) ||
        (with_scale && weight && ranges_touch(out, bytes, weight, bytes)) ||
        norm_inverse(x, weight, n, eps, with_scale, &inv) != 0)
        return -1;
    for (int i = 0; i < n; i++) {
        float y = x[i] * inv;
        if (with_scale) y = y * weight[i];
        out[i] = y;
    }
    return 0;
}

int orc_router_input(float *out, const float *state, const float *scale,
                     int hidden, float eps) {
    float inv;
    if (!out || !state || !scale || hidden < 1) return -1;
    size_t bytes = (size_t)hidden * 4;
    if ((out != state && ranges_touch(out, bytes, state, bytes)) ||
        ranges_touch(out, bytes, scale, bytes))
        return -1;
    for (int i = 0; i < hidden; i++)
        if (!isfinite(scale[i])) return -1;
    if (norm_inverse(state, NULL, hidden, eps, 0, &inv) != 0) return -1;
    float root = 1.0f / orc_sqrtf((float)hidden);
    for (int pass = 0; pass < 2; pass++)
        for (int i = 0; i < hidden; i++) {
            float y = state[i] * inv;
            y = y * scale[i];
            y = y * root;
            if (pass == 0) { if (!isfinite(y)) return -1; }
            else out[i] = y;
        }
    return 0;
}

int orc_residual_postnorm(float *out, const float *residual,
                          const float *branch, const float *weight, int n,
                          float eps) {
    float inv;
    if (!out || !residual || !branch || !weight || n < 1) return -1;
    size_t bytes = (size_t)n * 4;
    if (ranges_touch(out, bytes, residual, bytes) ||
        ranges_touch(out, bytes, branch, bytes) ||
        ranges_touch(out, bytes, weight, bytes))
        return -1;
    for (int i = 0; i < n; i++)
        if (!isfinite(residual[i])) return -1;
    if (norm_inverse(branch, weight, n, eps, 1, &inv) != 0) return -1;
    for (int pass = 0; pass < 2; pass++)
        for (int i = 0; i < n; i++) {
            float normalized = branch[i] * inv;
            normalized = normalized * weight[i];
            float y = residual[i] + normalized;
            if (pass == 0) { if (!isfinite(y)) return -1; }
            else out[i] = y;
        }
    return 0;
}

int orc_parallel_ffn_combine(float *out, const float *residual,
                             const float *dense, const float *routed,
                             const float *dense_post_weight,
                             const float *routed_post_weight,
                             const float *final_post_weight,
                             float layer_scalar, int n, float eps) {
    if (!out || !residual || !dense || !routed || !dense_post_weight ||
        !routed_post_weight || !final_post_weight || n < 1 ||
        !isfinite(layer_scalar))
        return -1;
    size_t bytes = (size_t)n * 4;
    const void *inputs[6] = {residual, dense, routed, dense_post_weight,
                             routed_post_weight, final_post_weight};
    for (int k = 0; k < 6; k++)
        if (ranges_touch(out, bytes, inputs[k], bytes)) return -1;
    for (int i = 0; i < n; i++)
        if (!isfinite(residual[i])) return -1;
    float *sum = (float *)malloc(2 * bytes);
    if (!sum) return -1;
    float *final = sum + n;
    int rc = -1;
    if (orc_rmsnorm(sum, dense, dense_post_weight, n, eps, 1) != 0 ||
        orc_rmsnorm(final, routed, routed_post_weight, n, eps, 1) != 0)
        goto done;
    for (int i = 0; i < n; i++) {
        float combined = sum[i] + final[i];
        if (!isfinite(combined)) goto done;
        sum[i] = combined;
    }
    if (orc_rmsnorm(final, sum, final_post_weight, n, eps, 1) != 0) goto done;
    for (int pass = 0; pass < 2; pass++)
        for (int i = 0; i < n; i++) {
            float y = residual[i] + final[i];
            y = y * layer_scalar;
            if (pass == 0) { if (!isfinite(y)) goto done; }
            else out[i] = y;
        }
    rc = 0;
done:
    free(sum);
    return rc;
}

int orc_softcap(float *logits, int n, float cap) {
    if (!logits || n < 1 || !(cap > 0.0f) || !isfinite(cap)) return -1;
    for (int i = 0; i < n; i++)
        if (!isfinite(logits[i])) return -1;
    for (int i = 0; i < n; i++) {
        float t = orc_tanhf(logits[i] / cap);
        logits[i] = cap * t;
    }
    return 0;
}

/* ------------------------------------------------------------------ */
/* routers                                                             */
/* ------------------------------------------------------------------ */

static int ranges_touch(const void *a, size_t na, const void *b, size_t nb) {
    uintptr_t pa = (uintptr_t)a, pb = (uintptr_t)b;
    return pa < pb + nb && pb < pa + na;
}

int orc_router_topk(const float *logits, const float *per_expert_scale,
                    int n_experts, int topk, int *selected, float *weights) {
    if (!logits || !per_expert_scale || !selected || !weights ||
        n_experts < 1 || topk < 1 || topk > n_experts)
        return -1;
    size_t in_bytes = (size_t)n_experts * 4u, out_bytes = (size_t)topk * 4u;
    if (ranges_touch(selected, out_bytes, weights, out_bytes) ||
        ranges_touch(selected, out_bytes, logits, in_bytes) ||
        ranges_touch(selected, out_bytes, per_expert_scale, in_bytes) ||
        ranges_touch(weights, out_bytes, logits, in_bytes) ||
        ranges_touch(weights, out_bytes, per_expert_scale, in_bytes))
        return -1;
    float peak = -INFINITY;
    for (int e = 0; e < n_experts; e++) {
        if (!isfinite(logits[e]) || !isfinite(per_expert_scale[e])) return -1;
        if (logits[e] > peak) peak = logits[e];
    }
    /* Descending list of the best logits so far; a later expert must be
     * strictly greater to pass an earlier one, so the lower index wins ties. */
    int held = 0;
    for (int j = 0; j < topk; j++) { selected[j] = -1; weights[j] = -INFINITY; }
    for (int e = 0; e < n_experts; e++) {
        int at = held;
        while (at > 0 && logits[e] > weights[at - 1]) at--;
        if (at >= topk) continue;
        int last = held < topk ? held : topk - 1;
        for (int j = last; j > at; j--) {
            selected[j] = selected[j - 1];
            weights[j] = weights[j - 1];
        }
        selected[at] = e;
        weights[at] = logits[e];
        if (held < topk) held++;
    }
    float all = 0.0f;
    for (int e = 0; e < n_experts; e++) all = all + orc_expf(logits[e] - peak);
    if (!(all > 0.0f) || !isfinite(all)) return -1;
    float chosen = 0.0f;
    for (int j = 0; j < topk; j++) {
        weights[j] = orc_expf(weights[j] - peak) / all;
        chosen = chosen + weights[j];
    }
    if (!(chosen > 0.0f) || !isfinite(chosen)) return -1;
    for (int j = 0; j < topk; j++) {
        float share = weights[j] / chosen;
        weights[j] = share * per_expert_scale[selected[j]];
    }
    return 0;
}

void orc_sort_selection(int *selected, float *weights, int topk) {
    /* Exchange sort ascending by expert id, weights carried along.  Ids are
     * distinct, so any correct sort gives the same arrangement. */
    for (int i = 0; i < topk; i++)
        for (int j = i + 1; j < topk; j++)
            if (selected[j] < selected[i]) {
                int ti = selected[i]; selected[i] = selected[j]; selected[j] = ti;
                float tw = weights[i]; weights[i] = weights[j]; weights[j] = tw;
            }
}

uint64_t orc_mix64(uint64_t x) {
    x += UINT64_C(0x9E3779B97F4A7C15);
    x = (x ^ (x >> 30)) * UINT64_C(0xBF58476D1CE4E5B9);
    x = (x ^ (x >> 27)) * UINT64_C(0x94D049BB133111EB);
    return x ^ (x >> 31);
}

static uint64_t mix3(uint64_t a, uint64_t b, uint64_t c) {
    return orc_mix64(a ^ orc_mix64(b * UINT64_C(0x100000001B3) + c));
}

int orc_router_fixture(int *idx, float *w, int n_experts, int topk,
                       uint64_t state, int layer, double locality) {
    if (!idx || !w || n_experts < 1 || topk < 1 || topk > n_experts) return -1;
    float *score = (float *)malloc((size_t)n_experts * sizeof(float));
    float *choice = (float *)malloc((size_t)n_experts * sizeof(float));
    char *taken = (char *)calloc((size_t)n_experts, 1);
    if (!score || !choice || !taken) {
        free(score); free(choice); free(taken);
        return -1;
    }
    for (int e = 0; e < n_experts; e++) {
        double plain = (double)(mix3(state, (uint64_t)layer, (uint64_t)e) &
                                0xFFFFFFu) / 16777216.0;
        double tilt = (double)(mix3(state ^ UINT64_C(0xB1A5), (uint64_t)layer,
                                    (uint64_t)e) & 0xFFFFFFu) / 16777216.0;
        double pick = plain + (tilt - 0.5) * 0.1;
        if (locality > 0.0) {
            double pop = 1.0 / (1.0 + (double)(e % 64));
            pick = plain * (1.0 + locality * pop);
        }
        score[e] = (float)plain;
        choice[e] = (float)pick;
    }
    for (int j = 0; j < topk; j++) {
        int best = -1;
        for (int e = 0; e < n_experts; e++)
            if (!taken[e] && (best < 0 || choice[e] > choice[best])) best = e;
        taken[best] = 1;
        idx[j] = best;
        w[j] = score[best];
    }
    free(score); free(choice); free(taken);
    return 0;
}

/* ------------------------------------------------------------------ */
/* routed expert FFN and MoE layer                                     */
/* ------------------------------------------------------------------ */

size_t orc_expert_proj_bytes(const OrcExpertGeometry *g) {
    size_t n = (size_t)g->hidden * (size_t)g->routed;
    return n / 2u + 2u * (n / ORC_GROUP) * 2u;
}

size_t orc_expert_slot_bytes(const OrcExpertGeometry *g) {
    return 3u * orc_expert_proj_bytes(g);
}

int orc_expert_ffn(const OrcExpertGeometry *g, const unsigned char *slot,
                   const float *input, float *gate, float *up, float *output) {
    if (!g || !slot || !input || !gate || !up || !output) return -1;
    size_t n = (size_t)g->hidden * (size_t)g->routed;
    size_t vals_bytes = n / 2u, meta_bytes = (n / ORC_GROUP) * 2u;
    size_t proj = orc_expert_proj_bytes(g);
    const unsigned char *wg = slot, *wu = slot + proj, *wd = slot + 2u * proj;
    if (orc_q4_matvec(wg, wg + vals_bytes, wg + vals_bytes + meta_bytes,
                      g->routed, g->hidden, input, gate) != 0 ||
        orc_q4_matvec(wu, wu + vals_bytes, wu + vals_bytes + meta_bytes,
                      g->routed, g->hidden, input, up) != 0)
        return -1;
    for (int i = 0; i < g->routed; i++)
        gate[i] = orc_gelu_tanh(gate[i]) * up[i];
    return orc_q4_matvec(wd, wd + vals_bytes, wd + vals_bytes + meta_bytes,
                         g->hidden, g->routed, gate, output);
}

typedef struct {
    const OrcExpertGeometry *g;
    const unsigned char *slot;
    const float *input;
    float *gate, *up, *output;
    int rc;
} ExpertCall;

typedef struct {
    ExpertCall *calls;
    int count, stride, first;
} ExpertLane;

static void *expert_lane_main(void *opaque) {
    ExpertLane *lane = (ExpertLane *)opaque;
    for (int i = lane->first; i < lane->count; i += lane->stride) {
        ExpertCall *c = &lane->calls[i];
        c->rc = orc_expert_ffn(c->g, c->slot, c->input, c->gate, c->up,
                               c->output);
    }
    return NULL;
}

/* Run `count` independent expert calls on up to `threads` threads. */
static int run_expert_calls(ExpertCall *calls, int count, int threads) {
    pthread_t tid[64];
    ExpertLane lane[64];
    int live[64];
    if (threads < 1) threads = 1;
    if (threads > 64) threads = 64;
    if (threads > count) threads = count;
    for (int t = 0; t < threads; t++) {
        lane[t].calls = calls; lane[t].count = count;
        lane[t].stride = threads; lane[t].first = t;
        live[t] = 0;
        if (threads > 1 &&
            pthread_create(&tid[t], NULL, expert_lane_main, &lane[t]) == 0)
            live[t] = 1;
        else
            expert_lane_main(&lane[t]);
    }
    for (int t = 0; t < threads; t++)
        if (live[t]) pthread_join(tid[t], NULL);
    for (int i = 0; i < count; i++)
        if (calls[i].rc != 0) return -1;
    return 0;
}

int orc_moe_decode_step(const OrcExpertGeometry *g, const unsigned char *pool,
                        int n_experts, int topk, const float *logits,
                        const float *per_expert_scale, const float *input,
                        int *selected, float *weights, float *expert_out,
                        float *output, int threads) {
    if (!g || !pool || !input || !selected || !weights || !output) return -1;
    if (orc_router_topk(logits, per_expert_scale, n_experts, topk, selected,
                        weights) != 0)
        return -1;
    orc_sort_selection(selected, weights, topk);
    size_t slot = orc_expert_slot_bytes(g);
    size_t H = (size_t)g->hidden, F = (size_t)g->routed;
    float *own = NULL;
    if (!expert_out) {
        own = (float *)malloc((size_t)topk * H * sizeof(float));
        if (!own) return -1;
        expert_out = own;
    }
    float *scratch = (float *)malloc((size_t)topk * 2u * F * sizeof(float));
    ExpertCall *calls = (ExpertCall *)calloc((size_t)topk, sizeof *calls);
    int rc = -1;
    if (scratch && calls) {
        for (int i = 0; i < topk; i++) {
            calls[i].g = g;
            calls[i].slot = pool + (size_t)selected[i] * slot;
            calls[i].input = input;
            calls[i].gate = scratch + (size_t)i * 2u * F;
            calls[i].up = calls[i].gate + F;
            calls[i].output = expert_out + (size_t)i * H;
        }
        rc = run_expert_calls(calls, topk, threads);
    }
    if (rc == 0) {
        for (size_t d = 0; d < H; d++) output[d] = 0.0f;
        for (int i = 0; i < topk; i++)
            for (size_t d = 0; d < H; d++) {
                float term = expert_out[(size_t)i * H + d] * weights[i];
                output[d] = output[d] + term;
            }
    }
    free(calls); free(scratch); free(own);
    return rc;
}

int orc_moe_group(const OrcExpertGeometry *g, const unsigned char *pool,
                  int n_experts, int topk, int batch, const int *selected,
                  const float *weights, const float *inputs, float *outputs,
                  int *group_rows, int threads) {
    if (!g || !pool || !selected || !weights || !inputs || !outputs ||
        batch < 1 || topk < 1 || n_experts < 1 || topk > n_experts)
        return -1;
    size_t H = (size_t)g->hidden, F = (size_t)g->routed;
    size_t picks = (size_t)batch * (size_t)topk;
    for (int t = 0; t < batch; t++)
        for (int k = 0; k < topk; k++) {
            size_t s = (size_t)t * (size_t)topk + (size_t)k;
            if (selected[s] < 0 || selected[s] >= n_experts ||
                !isfinite(weights[s]))
                return -1;
            for (int p = 0; p < k; p++)
                if (selected[(size_t)t * (size_t)topk + (size_t)p] ==
                    selected[s])
                    return -1;
        }
    /* Rows of a group are independent, so the values do not depend on the
     * grouping; the canonical order (expert, then token, then rank) only
     * fixes where each row sits in the grouped buffers. */
    if (group_rows) {
        for (int e = 0; e < n_experts; e++) group_rows[e] = 0;
        for (size_t s = 0; s < picks; s++) group_rows[selected[s]]++;
    }
    float *pick_out = (float *)malloc(picks * H * sizeof(float));
    float *scratch = (float *)malloc(picks * 2u * F * sizeof(float));
    ExpertCall *calls = (ExpertCall *)calloc(picks, sizeof *calls);
    int rc = -1;
    size_t slot = orc_expert_slot_bytes(g);
    if (pick_out && scratch && calls) {
        for (size_t s = 0; s < picks; s++) {
            calls[s].g = g;
            calls[s].slot = pool + (size_t)selected[s] * slot;
            calls[s].input = inputs + (s / (size_t)topk) * H;
            calls[s].gate = scratch + s * 2u * F;
            calls[s].up = calls[s].gate + F;
            calls[s].output = pick_out + s * H;
        }
        rc = run_expert_calls(calls, (int)picks, threads);
    }
    if (rc == 0)
        for (int t = 0; t < batch; t++) {
            float *out = outputs + (size_t)t * H;
            for (size_t d = 0; d < H; d++) out[d] = 0.0f;
            for (int k = 0; k < topk; k++) {
                size_t s = (size_t)t * (size_t)topk + (size_t)k;
                for (size_t d = 0; d < H; d++) {
                    float term = pick_out[s * H + d] * weights[s];
                    out[d] = out[d] + term;
                }
            }
        }
    free(calls); free(scratch); free(pick_out);
    return rc;
}

/* ------------------------------------------------------------------ */
/* feed-forward half of a decoder layer                                */
/* ------------------------------------------------------------------ */

int orc_ffn_block(const OrcFfnLayer *L, const float *residual, float *output,
                  int *selected, float *weights, int threads) {
    if (!L || !residual || !output || L->hidden < 1 || L->dense < 1 ||
        L->topk < 1 || L->topk > L->n_experts)
        return -1;
    size_t H = (size_t)L->hidden, D = (size_t)L->dense;
    size_t E = (size_t)L->n_experts, K = (size_t)L->topk;
    float *buf = (float *)malloc((4 * H + 2 * D + E + K) * sizeof(float));
    int *sel = (int *)malloc(K * sizeof(int));
    int rc = -1;
    if (!buf || !sel) goto done;
    float *norm = buf, *dense_out = buf + H, *routed_out = buf + 2 * H;
    float *router_in = buf + 3 * H, *gate = buf + 4 * H, *up = gate + D;
    float *logits = up + D, *w = logits + E;
    OrcExpertGeometry g = {L->hidden, L->routed};

    if (orc_rmsnorm(norm, residual, L->pre_norm, L->hidden, L->eps, 1) != 0 ||
        orc_q4_matvec_threads(L->dense_gate[0], L->dense_gate[1], L->dense_gate[2], L->dense, L->hidden, norm, gate,
                              threads) != 0 ||
        orc_q4_matvec_threads(L->dense_up[0], L->dense_up[1], L->dense_up[2], L->dense, L->hidden, norm, up,
                              threads) != 0)
        goto done;
    for (size_t i = 0; i < D; i++) gate[i] = orc_gelu_tanh(gate[i]) * up[i];
    if (orc_q4_matvec_threads(L->dense_down[0], L->dense_down[1], L->dense_down[2], L->hidden, L->dense, gate,
                              dense_out, threads) != 0)
        goto done;

    if (orc_router_input(router_in, residual, L->router_scale, L->hidden, L->eps) != 0) goto done;
    orc_q8_matvec(L->router[0], L->router[1], L->router[2], L->n_experts, L->hidden, router_in, logits);
    if (orc_rmsnorm(norm, residual, L->pre_norm_2, L->hidden, L->eps, 1) != 0) goto done;
    if (orc_moe_decode_step(&g, L->pool, L->n_experts, L->topk, logits, L->per_expert_scale, norm, sel, w, NULL,
                            routed_out, threads) != 0)
        goto done;
    if (orc_parallel_ffn_combine(output, residual, dense_out, routed_out, L->post_norm_1, L->post_norm_2,
                                 L->post_norm, L->layer_scalar, L->hidden, L->eps) != 0)
        goto done;
    if (selected) memcpy(selected, sel, K * sizeof(int));
    if (weights) memcpy(weights, w, K * sizeof(float));
    rc = 0;
done:
    free(buf); free(sel);
    return rc;
}
