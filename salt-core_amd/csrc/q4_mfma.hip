// Prefill-sized affine-Q4 matmul on the MFMA units (tolerance class).
//
// When many tokens meet one weight matrix the work is a dense contraction and
// the 32-chain order of the decode kernels cannot be kept at matrix-core speed.
// This kernel computes Y[token][row] = sum_c (q*s + b)[row][c] * x[token][c]
// with fp32-level accuracy but in a different summation order; callers opt in
// and are told so (the engine's bit-exact path remains the tiled kernels).
//
// How the affine weights reach the matrix cores without losing bits:
//  * per 64-column scale group,  sum_c (q s + b) x = s * sum_c q x + b * sum_c x.
//    The integer codes are exact in bf16, so only sum_c q x goes through MFMA
//    per group; the scale is applied per group in fp32 on the VALU.
//  * a nibble becomes the fp16 value 16 + q with two bit operations per pair
//    ((w shifted) & 0x03C003C0 | 0x4C004C00); the surplus 16 * s * sum_c x joins
//    the bias term.
//  * the activation row is scaled by a power of two that puts its largest
//    magnitude in [2^13, 2^14) and split into two fp16 planes, x * 2^k = hi + lo
//    (each rounded to nearest: 23 significant bits, |x 2^k - hi - lo| <= 2^-22
//    of the element's own magnitude, or 2^-25 of the scaled row for elements so
//    small that lo is subnormal); each plane is an exact MFMA operand,
//    accumulation is fp32, and the power of two leaves with the store.
//  * the bias term sum_g (b_g - 16 s_g) * X_g (X_g = the group sums of x) is
//    itself a small contraction over the groups; b and s are bf16, so it runs
//    on the matrix cores once per tile before the main loop, with X_g split
//    into three bf16 planes (v = hi + mid + lo to 2^-24).
//
// Tiling: a workgroup of four waves computes 64 tokens x 128 weight rows, each
// wave 32 tokens x 64 rows as two 32 x 32 blocks of v_mfma_f32_32x32x16_f16
// that share the token operand (tokens are the M rows, weight rows the N
// columns, so a lane owns one weight row per block and needs one scale per
// group).  Per group the planes, the packed codes and the scales are staged in
// one of two LDS stages, the next group's loads in flight during the matrix
// work, one barrier per group.  Inside every aligned run of eight columns the
// planes are stored in the order 0,4,1,5,2,6,3,7, which is the order the pair
// extraction above yields the codes in.
#include "device_math.h"
#include "mi355_internal.h"

#include <stddef.h>
#include <type_traits>

namespace mi355 {
namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
constexpr int X_PLANES = 2;                // fp16 planes of the scaled activation
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef const uint64_t __attribute__((address_space(4))) *uniform_u64_ptr;
typedef const u32x4 __attribute__((address_space(1))) *global_u128_ptr;
typedef const uint16_t __attribute__((address_space(1))) *global_u16_ptr;
typedef const float __attribute__((address_space(1))) *global_f32_ptr;

constexpr int TM = MFMA_TM;                 // tokens per workgroup; weight rows per workgroup: 64 * NBW
constexpr int X_PITCH = 144;               // bytes per staged token row of one plane: 64 halves + 16 pad
constexpr int W_PITCH = 36;                // bytes per staged weight row of one group: 32 + 4 pad
constexpr int XS_BYTES = X_PLANES * TM * X_PITCH;
constexpr int G_PITCH = 48;                // bias pass: bytes per staged row of 16 bf16: 32 + 16 pad
constexpr int XG_BYTES = 3 * TM * G_PITCH;

// LDS layout of one stage for a tile of TN weight rows
template <int TN> struct Stage {
    static constexpr int WS_OFF = XS_BYTES;                        // codes [TN][W_PITCH]
    static constexpr int SC_OFF = WS_OFF + TN * W_PITCH;           // float scale[TN]
    static constexpr int BYTES = (SC_OFF + TN * 4 + 15) & ~15;
    static_assert(XG_BYTES + 2 * TN * G_PITCH <= 2 * BYTES, "the bias pass reuses the staging memory");
};

static_assert(sizeof(MfmaJob) == 64, "find_job reads a job record as eight 64-bit words");

__device__ __forceinline__ MfmaJob find_job(const MfmaLaunch &L, int tile) {
    if (L.table == nullptr) return L.one;
    const uniform_u64_ptr words = (uniform_u64_ptr)(uintptr_t)L.table;
    const int njobs = L.njobs_dev ? *(const int __attribute__((address_space(4))) *)(uintptr_t)L.njobs_dev : L.njobs;
    int lo = 0, hi = njobs - 1;
    while (lo < hi) {
        const int mid = (lo + hi + 1) >> 1;
        if ((int)(uint32_t)words[8 * mid + 7] <= tile) lo = mid; else hi = mid - 1;
    }
    const uniform_u64_ptr rec = words + 8 * lo;
    MfmaJob job;
    job.vals = (const uint8_t *)rec[0];
    job.scales = (const uint8_t *)rec[1];
    job.biases = (const uint8_t *)rec[2];
    job.planes = (const uint16_t *)rec[3];
    job.xsum = (const float *)rec[4];
    job.y = (float *)rec[5];
    job.tokens = (int)(uint32_t)rec[6];
    job.rows = (int)(rec[6] >> 32);
    job.tile0 = (int)(uint32_t)rec[7];
    job.row_base = (int)(rec[7] >> 32);
    return job;
}

__device__ __forceinline__ float bf16_to_f32(uint32_t half) { return __uint_as_float(half << 16); }

// Eight nibbles -> eight fp16 values 16 + q, in the column order 0,4,1,5,2,6,3,7.
// (a & mask) | bits in one instruction; the three-operand form takes no
// literals, so the mask travels in a scalar register and the bits in a vector one.
__device__ __forceinline__ uint32_t and_or(uint32_t a, uint32_t mask, uint32_t bits) {
    uint32_t r;
    asm("v_and_or_b32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "s"(mask), "v"(bits));
    return r;
}

__device__ __forceinline__ f16x8 codes_to_f16(uint32_t w, uint32_t mask, uint32_t sixteen) {
    u32x4 r;                                             // a code's four bits land on mantissa bits 6..9 of 16.0
    r.x = and_or((w << 6), mask, sixteen);               // columns 0 and 4
    r.y = and_or((w << 2), mask, sixteen);               // 1 and 5
    r.z = and_or((w >> 2), mask, sixteen);               // 2 and 6
    r.w = and_or((w >> 6), mask, sixteen);               // 3 and 7
    return __builtin_bit_cast(f16x8, r);
}

// 2^-k <-> 2^k for a float that is a power of two (normal range)
__device__ __forceinline__ float reciprocal_power_of_two(float p) {
    return __uint_as_float((254u - ((__float_as_uint(p) >> 23) & 0xffu)) << 23);
}

__device__ __forceinline__ uint32_t f32_to_bf16_rne(float v) {
    const uint32_t bits = __float_as_uint(v);
    return (bits + 0x7FFFu + ((bits >> 16) & 1u)) >> 16;
}

// v = hi + mid + lo, each a bf16 (bit patterns in the low halves)
__device__ __forceinline__ void split3(float v, uint32_t &h, uint32_t &m, uint32_t &l) {
    h = f32_to_bf16_rne(v);
    const float r1 = v - bf16_to_f32(h);
    m = f32_to_bf16_rne(r1);
    const float r2 = r1 - bf16_to_f32(m);
    l = f32_to_bf16_rne(r2);
}

// One scale group of one wave: NB blocks of 32 rows against the wave's 32 tokens.
template <int NB, int NBW>
__device__ __forceinline__ void group_product(const uint8_t *cur, int wm, int wn, int l32, int half,
                                              f32x16 (&acc)[NBW]) {
    using S = Stage<64 * NBW>;
    const f32x16 zero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
    uint32_t sixteen;                                   // two fp16 values 16.0, kept in a vector register
    asm("v_mov_b32 %0, 0x4C004C00" : "=v"(sixteen));
    const uint8_t *wrow = cur + S::WS_OFF + (wn * 32 * NBW + l32) * W_PITCH + half * 4;
    const uint8_t *xrow = cur + (wm * 32 + l32) * X_PITCH + half * 16;
    const float *sc = reinterpret_cast<const float *>(cur + S::SC_OFF) + wn * 32 * NBW + l32;
    // The token operand of the whole group stays in registers; the row blocks
    // then run two at a time so that only two partial products are live.
    f16x8 a[4][X_PLANES];
#pragma unroll
    for (int ks = 0; ks < 4; ++ks)
#pragma unroll
        for (int plane = 0; plane < X_PLANES; ++plane)
            a[ks][plane] = __builtin_bit_cast(
                f16x8, *reinterpret_cast<const u32x4 *>(xrow + plane * (TM * X_PITCH) + ks * 32));
#pragma unroll
    for (int nb0 = 0; nb0 < NB; nb0 += 2) {
        constexpr int PAIR_MAX = 2;
        const int pair = NB - nb0 < PAIR_MAX ? NB - nb0 : PAIR_MAX;
        f32x16 part[PAIR_MAX];
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) {
            f16x8 b[PAIR_MAX];
#pragma unroll
            for (int k = 0; k < PAIR_MAX; ++k)
                if (k < pair)
                    b[k] = codes_to_f16(*reinterpret_cast<const uint32_t *>(wrow + (nb0 + k) * 32 * W_PITCH + ks * 8),
                                        0x03C003C0u, sixteen);
#pragma unroll
            for (int plane = 0; plane < X_PLANES; ++plane)
#pragma unroll
                for (int k = 0; k < PAIR_MAX; ++k)
                    if (k < pair)
                        part[k] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[ks][plane], b[k],
                                                                         (ks | plane) ? part[k] : zero, 0, 0, 0);
        }
#pragma unroll
        for (int k = 0; k < PAIR_MAX; ++k)
            if (k < pair) {
                const float s = sc[(nb0 + k) * 32];
#pragma unroll
                for (int i = 0; i < 16; ++i) acc[nb0 + k][i] = __builtin_fmaf(s, part[k][i], acc[nb0 + k][i]);
            }
    }
}

// NBW = 32-row blocks per wave: the workgroup's tile is 64 tokens x 64 * NBW rows.
template <int NBW>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2)))
void q4_mfma_kernel(const MfmaLaunch L) {
    constexpr int TN = 64 * NBW;
    using S = Stage<TN>;
    constexpr int STAGE_BYTES = S::BYTES;
    // two stages of { planes [2][64 tokens], codes [TN rows], scales [TN] }
    __shared__ __attribute__((aligned(16))) uint8_t stage[2 * STAGE_BYTES];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave >> 1, wn = wave & 1;       // wave tile: tokens wm*32.., rows wn*32*NBW.. (NBW 32-row blocks)
    const int l32 = lane & 31, half = lane >> 5;

    if (L.total_tiles_dev &&
        (int)blockIdx.x >= *(const int __attribute__((address_space(4))) *)(uintptr_t)L.total_tiles_dev)
        return;                                     // uniform: the whole workgroup leaves
    const MfmaJob job = find_job(L, blockIdx.x);
    const int C = L.cols, ngrp = C >> 6;
    const int ntiles = (job.rows + TN - 1) / TN;
    const int t = blockIdx.x - job.tile0;
    const int tok0 = (t / ntiles) * TM, row0 = (t % ntiles) * TN;
    const int toks_here = job.tokens - tok0 < TM ? job.tokens - tok0 : TM;
    const int rows_here = job.rows - row0 < TN ? job.rows - row0 : TN;

    // Token t of the job is row (tok0 + t) of the planes, or, with a map, row
    // row_map[row_base + tok0 + t] / map_divisor (the grouped MoE gather).
    const int *row_map = L.row_map;
    auto source_row = [&](int tok) -> uint32_t {
        const int tc = tok < toks_here ? tok : toks_here - 1;
        return row_map ? (uint32_t)(row_map[job.row_base + tok0 + tc] / L.map_divisor) : (uint32_t)(tok0 + tc);
    };

    // staging geometry of this thread
    // planes: 2 * 64 tokens * 8 segments of 16 bytes = 1024 pieces, 4 per thread
    constexpr int XP = X_PLANES * TM * 8 / 256;
    const global_u16_ptr planes = (global_u16_ptr)(uintptr_t)job.planes;
    uint32_t x_src[XP], x_dst[XP];                  // element offsets: the planes of one launch stay below 2^32 elements
#pragma unroll
    for (int i = 0; i < XP; ++i) {
        const int p = tid + i * 256;
        const int plane = p >> 9, tok = (p >> 3) & 63, seg = p & 7;
        x_src[i] = (uint32_t)plane * (uint32_t)L.plane_stride + source_row(tok) * (uint32_t)C + seg * 8;
        x_dst[i] = plane * (TM * X_PITCH) + tok * X_PITCH + seg * 16;
    }
    // codes: TN rows * 2 pieces of 16 bytes, NBW / 2 per thread
    constexpr int WP = NBW / 2;
    const int w_half = tid & 1;
    global_u128_ptr w_src[WP];
    uint32_t w_dst[WP];
#pragma unroll
    for (int i = 0; i < WP; ++i) {
        const int row = (tid >> 1) + i * 128;
        const int rc = row < rows_here ? row : rows_here - 1;
        w_src[i] = (global_u128_ptr)((uintptr_t)job.vals + (size_t)(row0 + rc) * (C >> 1) + w_half * 16);
        w_dst[i] = S::WS_OFF + row * W_PITCH + w_half * 16;
    }
    // scales: threads 0..TN-1
    const int m_row = tid & (TN - 1);
    const int m_rc = m_row < rows_here ? m_row : rows_here - 1;
    const global_u16_ptr scales = (global_u16_ptr)(uintptr_t)job.scales + (size_t)(row0 + m_rc) * ngrp;

    // Loads travel through registers; two sets are in flight so that a load has
    // two groups of matrix work (of both workgroups on the compute unit) to land.
    struct Loads { u32x4 x[XP], w[WP]; uint32_t s; };
    auto issue = [&](int g, Loads &r) {
#pragma unroll
        for (int i = 0; i < XP; ++i) r.x[i] = *(global_u128_ptr)(planes + x_src[i] + (uint32_t)g * 64u);
#pragma unroll
        for (int i = 0; i < WP; ++i) r.w[i] = w_src[i][g * 2];
        if (tid < TN) r.s = scales[g];
    };
    auto commit = [&](uint8_t *base, const Loads &r) {
#pragma unroll
        for (int i = 0; i < XP; ++i) *reinterpret_cast<u32x4 *>(base + x_dst[i]) = r.x[i];
#pragma unroll
        for (int i = 0; i < WP; ++i) {
            uint32_t *dst = reinterpret_cast<uint32_t *>(base + w_dst[i]);
            dst[0] = r.w[i].x; dst[1] = r.w[i].y; dst[2] = r.w[i].z; dst[3] = r.w[i].w;
        }
        if (tid < TN) reinterpret_cast<float *>(base + S::SC_OFF)[m_row] = bf16_to_f32(r.s);
    };

    const f32x16 zero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
    f32x16 acc[NBW];
#pragma unroll
    for (int nb = 0; nb < NBW; ++nb) acc[nb] = zero;

    // ---- bias pass: acc[tok][row] = sum_g (b[row][g] - 16 s[row][g]) * X[tok][g]
    {
        const global_f32_ptr xsum = (global_f32_ptr)(uintptr_t)job.xsum;
        const int xg_tok = tid >> 2, xg_g = (tid & 3) * 4;
        const size_t xg_row = (size_t)source_row(xg_tok) * ngrp;
        const global_u16_ptr all_scales = (global_u16_ptr)(uintptr_t)job.scales;
        const global_u16_ptr all_biases = (global_u16_ptr)(uintptr_t)job.biases;
        // Two 32-row blocks per pass keep the four partial products in registers.
#pragma unroll 1
        for (int pass = 0; pass < NBW / 2; ++pass) {
            f32x16 tb[2] = {zero, zero}, ts[2] = {zero, zero};
            for (int g0 = 0; g0 < ngrp; g0 += 16) {
                uint32_t h[4], m[4], l[4];
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const int g = g0 + xg_g + j;
                    const float v = g < ngrp ? xsum[xg_row + g] : 0.0f;
                    split3(v, h[j], m[j], l[j]);
                }
                __syncthreads();                                // the previous step's operands have been read
                uint8_t *xgp = stage + xg_tok * G_PITCH + xg_g * 2;
                *reinterpret_cast<uint2 *>(xgp) = make_uint2(h[0] | h[1] << 16, h[2] | h[3] << 16);
                *reinterpret_cast<uint2 *>(xgp + TM * G_PITCH) = make_uint2(m[0] | m[1] << 16, m[2] | m[3] << 16);
                *reinterpret_cast<uint2 *>(xgp + 2 * TM * G_PITCH) = make_uint2(l[0] | l[1] << 16, l[2] | l[3] << 16);
                // (bias, scale) bits of 16 groups for every row of the tile: item = array * TN + row
                for (int item = tid; item < 2 * TN; item += 256) {
                    const int arr = item / TN, row = item % TN;
                    const int rc = row < rows_here ? row : rows_here - 1;
                    const global_u16_ptr src = (arr ? all_scales : all_biases) + (size_t)(row0 + rc) * ngrp;
                    const bool present = arr || job.biases;
                    uint32_t *bsp = reinterpret_cast<uint32_t *>(stage + XG_BYTES + item * G_PITCH);
#pragma unroll
                    for (int j = 0; j < 8; ++j) {
                        const int g = g0 + 2 * j;
                        const uint32_t lo = (present && g < ngrp) ? (uint32_t)src[g] : 0u;
                        const uint32_t hi = (present && g + 1 < ngrp) ? (uint32_t)src[g + 1] : 0u;
                        bsp[j] = lo | hi << 16;
                    }
                }
                __syncthreads();
                {
                    const uint8_t *arow = stage + (wm * 32 + l32) * G_PITCH + half * 16;
                    const uint8_t *brow = stage + XG_BYTES + (wn * 32 * NBW + pass * 64 + l32) * G_PITCH + half * 16;
#pragma unroll
                    for (int plane = 0; plane < 3; ++plane) {
                        const bf16x8 a = __builtin_bit_cast(bf16x8, *reinterpret_cast<const u32x4 *>(arow + plane * TM * G_PITCH));
#pragma unroll
                        for (int nb = 0; nb < 2; ++nb) {
                            const bf16x8 bb = __builtin_bit_cast(bf16x8, *reinterpret_cast<const u32x4 *>(brow + nb * 32 * G_PITCH));
                            const bf16x8 sb = __builtin_bit_cast(
                                bf16x8, *reinterpret_cast<const u32x4 *>(brow + (TN + nb * 32) * G_PITCH));
                            tb[nb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, bb, tb[nb], 0, 0, 0);
                            ts[nb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, sb, ts[nb], 0, 0, 0);
                        }
                    }
                }
            }
#pragma unroll
            for (int nb = 0; nb < 2; ++nb)
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    const float v = __builtin_fmaf(-16.0f, ts[nb][i], tb[nb][i]);
                    if (NBW == 2 || pass == 0) acc[nb][i] = v; else acc[(NBW > 2 ? 2 : 0) + nb][i] = v;
                }
        }
        __syncthreads();
    }

    // The main loop works on x * 2^k (k per token, chosen by the split): the bias term joins it at that scale and
    // the power of two leaves at the store.  A token's 2^-k lies at the head of its row of the third plane.
    auto token_scale = [&](int i) -> float {
        const int tok = wm * 32 + (i >> 2) * 8 + half * 4 + (i & 3);
        return *(const float __attribute__((address_space(1))) *)(uintptr_t)(
            job.planes + 2 * (size_t)L.plane_stride + (size_t)source_row(tok) * (size_t)C);
    };
#pragma unroll
    for (int i = 0; i < 16; ++i) {
        const float up = reciprocal_power_of_two(token_scale(i));
#pragma unroll
        for (int nb = 0; nb < NBW; ++nb) acc[nb][i] = acc[nb][i] * up;
    }

    // ---- main loop: acc += s[row][g] * sum_{c in g} (16 + q[row][c]) * x[tok][c] * 2^k
    // Row blocks past the end of the matrix are computed on clamped rows and
    // dropped at the store: one instantiation of the loop keeps the
    // accumulators in place and the register count inside the budget.
    {
        Loads even, odd;
        even.s = 0; odd.s = 0;
        uint8_t *stage0 = stage, *stage1 = stage + STAGE_BYTES;
        issue(0, even);
        if (ngrp > 1) issue(1, odd);
        commit(stage0, even);
        __syncthreads();
        for (int g = 0; g < ngrp; g += 2) {
            if (g + 2 < ngrp) issue(g + 2, even);
            group_product<NBW, NBW>(stage0, wm, wn, l32, half, acc);
            if (g + 1 < ngrp) commit(stage1, odd);
            __syncthreads();
            if (g + 1 >= ngrp) break;
            if (g + 3 < ngrp) issue(g + 3, odd);
            group_product<NBW, NBW>(stage1, wm, wn, l32, half, acc);
            if (g + 2 < ngrp) commit(stage0, even);
            __syncthreads();
        }
    }

    float __attribute__((address_space(1))) *y = (float __attribute__((address_space(1))) *)(uintptr_t)job.y;
    float down[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) down[i] = token_scale(i);
#pragma unroll
    for (int nb = 0; nb < NBW; ++nb) {
        const int row = wn * 32 * NBW + nb * 32 + l32;
        if (row < rows_here) {
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                const int tok = wm * 32 + (i >> 2) * 8 + half * 4 + (i & 3);
                if (tok < toks_here) y[(size_t)(tok0 + tok) * job.rows + row0 + row] = acc[nb][i] * down[i];
            }
        }
    }
}

// fp32 rows -> two fp16 planes of the row scaled by a power of two (columns permuted inside every run of eight, see
// the top of the file), the row's 2^-k at the head of its row of a third plane, and the per-64-column sums of the
// unscaled values.  Row r of the output is row row_map[r] / map_divisor of the input when a map is given (the
// grouped MoE gather).  One workgroup per row: the scale needs the row's largest magnitude.
// With GATED the value split is gelu_tanh(gate) * x (the expert activation, reference gemma4_text.c:8749-9137
// "down input"), so the activations never make a round trip through memory in fp32.
constexpr int SPLIT_MAX_ITEMS = 4;          // eight columns per item and thread: rows of up to 8192 columns

template <bool GATED>
__global__ __launch_bounds__(256) void x_split_kernel(const float *__restrict__ x, const float *__restrict__ gate,
                                                      const int *__restrict__ row_map, int map_divisor, int x_stride,
                                                      int rows, int cols, uint16_t *__restrict__ planes,
                                                      size_t plane_stride, float *__restrict__ xsum) {
    __shared__ uint32_t wave_top[4];
    const int row = blockIdx.x;
    const int src_row = row_map ? row_map[row] / map_divisor : row;
    float v[SPLIT_MAX_ITEMS][8];
    uint32_t top = 0u;                              // largest magnitude as a bit pattern: a NaN or an infinity wins it
#pragma unroll
    for (int it = 0; it < SPLIT_MAX_ITEMS; ++it) {
        const int c0 = (it * 256 + (int)threadIdx.x) * 8;
#pragma unroll
        for (int j = 0; j < 8; ++j) v[it][j] = 0.0f;
        if (c0 < cols) {
            const float4 *src = reinterpret_cast<const float4 *>(x + (size_t)src_row * x_stride + c0);
            const float4 a = src[0], b = src[1];
            v[it][0] = a.x; v[it][1] = a.y; v[it][2] = a.z; v[it][3] = a.w;
            v[it][4] = b.x; v[it][5] = b.y; v[it][6] = b.z; v[it][7] = b.w;
            if (GATED) {
                const float4 *gsrc = reinterpret_cast<const float4 *>(gate + (size_t)src_row * x_stride + c0);
                const float4 ga = gsrc[0], gb = gsrc[1];
                const float gv[8] = {ga.x, ga.y, ga.z, ga.w, gb.x, gb.y, gb.z, gb.w};
#pragma unroll
                for (int j = 0; j < 8; ++j) v[it][j] = det_gelu_tanh(gv[j]) * v[it][j];
            }
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const uint32_t mag = __float_as_uint(v[it][j]) & 0x7fffffffu;
                top = top > mag ? top : mag;
            }
        }
    }
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
        const uint32_t other = (uint32_t)__shfl_xor((int)top, d, 64);
        top = top > other ? top : other;
    }
    if ((threadIdx.x & 63) == 0) wave_top[threadIdx.x >> 6] = top;
    __syncthreads();
    top = wave_top[0];
#pragma unroll
    for (int w = 1; w < 4; ++w) top = top > wave_top[w] ? top : wave_top[w];
    // top in [2^E, 2^(E+1)) -> x * 2^(13 - E) in [2^13, 2^14); rows of zeros or tiny values are pinned
    int eb = (int)(top >> 23);
    eb = eb < 14 ? 14 : (eb > 253 ? 253 : eb);
    const float up = __uint_as_float((uint32_t)(267 - eb) << 23);          // 2^(13 - E)
    const float down = __uint_as_float((uint32_t)(eb - 13) << 23);         // 2^(E - 13)
    if (threadIdx.x == 0) *reinterpret_cast<float *>(planes + 2 * plane_stride + (size_t)row * cols) = down;
#pragma unroll
    for (int it = 0; it < SPLIT_MAX_ITEMS; ++it) {
        const int c0 = (it * 256 + (int)threadIdx.x) * 8;
        const bool live = c0 < cols;
        uint32_t hi[4], lo[4];
        float sum = 0.0f;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const float scaled = v[it][j] * up;
            const _Float16 h = (_Float16)scaled;
            const _Float16 l = (_Float16)(scaled - (float)h);
            const uint32_t hb = __builtin_bit_cast(uint16_t, h), lb = __builtin_bit_cast(uint16_t, l);
            const int k = j & 3;                           // dword k holds columns k (low half) and k + 4 (high half)
            if (j & 4) { hi[k] |= hb << 16; lo[k] |= lb << 16; }
            else { hi[k] = hb; lo[k] = lb; }
            sum += v[it][j];
        }
        // eight lanes cover one 64-column group
        sum += __shfl_xor(sum, 1, 64);
        sum += __shfl_xor(sum, 2, 64);
        sum += __shfl_xor(sum, 4, 64);
        if (live) {
            uint16_t *dst = planes + (size_t)row * cols + c0;
            *reinterpret_cast<uint4 *>(dst) = make_uint4(hi[0], hi[1], hi[2], hi[3]);
            *reinterpret_cast<uint4 *>(dst + plane_stride) = make_uint4(lo[0], lo[1], lo[2], lo[3]);
            if ((threadIdx.x & 7) == 0) xsum[(size_t)row * (cols >> 6) + (c0 >> 6)] = sum;
        }
    }
}

}  // namespace

int mfma_tile_rows(int blocks_per_wave) { return 64 * blocks_per_wave; }

int mfma_tiles(int tokens, int rows, int blocks_per_wave) {
    const int tn = mfma_tile_rows(blocks_per_wave);
    return ((tokens + TM - 1) / TM) * ((rows + tn - 1) / tn);
}

// Blocks of 32 rows per wave.  Four (a 64 x 256 tile) halves the LDS and cache
// traffic per matrix instruction but measured no faster than two: on this
// device the matrix instructions and the other vector instructions of a SIMD
// do not overlap, so the kernel is bound by their sum, not by data movement.
int mfma_blocks_per_wave(long long wide_tiles) {
    (void)wide_tiles;
    return 2;
}

int q4_mfma_launch(const MfmaLaunch &launch, hipStream_t stream) {
    MfmaLaunch L = launch;
    if (L.cols < 64 || (L.cols & 63)) return -1;
    if (L.table == nullptr) {                   // one job: the tiling is chosen here
        if (L.blocks_per_wave == 0) L.blocks_per_wave = mfma_blocks_per_wave(mfma_tiles(L.one.tokens, L.one.rows, 4));
        L.one.tile0 = 0;
        L.total_tiles = mfma_tiles(L.one.tokens, L.one.rows, L.blocks_per_wave);
    }
    if (3 * (unsigned long long)L.plane_stride >= (1ull << 32)) return -1;      // 32-bit element offsets in the kernel
    if (L.total_tiles < 1 || L.blocks_per_wave != 2 || (L.row_map && L.map_divisor < 1))
        return -1;
    hipLaunchKernelGGL(q4_mfma_kernel<2>, dim3(L.total_tiles), dim3(256), 0, stream, L);
    return hipGetLastError() == hipSuccess ? 0 : -1;
}

int x_split_launch(const float *x, const float *gate, const int *row_map, int map_divisor, int x_stride, int rows,
                   int cols, uint16_t *planes, size_t plane_stride, float *xsum, hipStream_t stream) {
    if (rows < 1 || cols < 64 || (cols & 63) || cols > SPLIT_MAX_ITEMS * 256 * 8) return -1;
    const dim3 grid(rows);
    if (gate)
        hipLaunchKernelGGL(x_split_kernel<true>, grid, dim3(256), 0, stream, x, gate, row_map, map_divisor, x_stride,
                           rows, cols, planes, plane_stride, xsum);
    else
        hipLaunchKernelGGL(x_split_kernel<false>, grid, dim3(256), 0, stream, x, gate, row_map, map_divisor, x_stride,
                           rows, cols, planes, plane_stride, xsum);
    return hipGetLastError() == hipSuccess ? 0 : -1;
}


}  // namespace mi355
