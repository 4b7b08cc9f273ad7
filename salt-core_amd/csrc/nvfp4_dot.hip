// NVFP4 matvec for gfx950, tolerance class: the HBM-bound decode kernel.
//
// The reference matvec (src/nvfp4.c:228-256) first quantises the activation to NVFP4 itself (group-16 Q/DQ,
// nvfp4.c:82-130) and then multiplies by the dequantised activation.  Both operands of every product are therefore an
// E2M1 code times a per-16-column factor:
//
//     y[r] = sum over 16-column blocks B of   (e4m3(s[r][B]) * wg) * (xs[B] / g)  *  sum_{c in B} e2m1(w[r][c]) * e2m1(xq[c])
//
// The inner sums are small multiples of 1/4 (at most 16 * 36): v_mfma_f32_32x32x64_f8f6f4 takes the packed codes of
// both sides as they are (no unpacking, no conversion) and adds them exactly.  The matrix instruction is used as a
// bank of dot-product units: its N side holds 32 weight rows, its K side 32 columns (two blocks) of each of two
// strips of the row, its M side one row per (token, strip, block) whose other columns are zero codes, which keeps the
// blocks' sums apart.  What remains per (row, block, token) is one E4M3 decode, two multiplies and a fused
// multiply-add; the activation codes are chosen with the reference's own rounding (closed-form encoders), so the
// only difference from the reference is the order and the rounding of the fp32 sum over the blocks.  Stated bound
// (tests): |y - y_ref| <= 2^-20 * sum_c |w_c x_c| per output.  A non-finite activation is rejected like the
// reference does: the status word becomes -1 and nothing is published for that job.
//
// Data movement is the affine-Q4 kernel's (dot_common.h, q4_dot.hip): 8 KiB steps straight into LDS, the lane's
// E4M3 scales of the whole block fetched once into registers and picked by register indexing.
#include "dot_common.h"
#include "nvfp4_device.h"

#include <stdio.h>

namespace mi355 {
namespace {

typedef int v8i __attribute__((ext_vector_type(8)));
typedef float v16f __attribute__((ext_vector_type(16)));

constexpr int FP4_ZERO_BYTES = 512;          // what lanes without activation codes read instead

__device__ __forceinline__ Fp4Job fp4_dot_find_job(const Fp4DotLaunch &L, int wg) {
    if (L.table == nullptr) return L.one;
    const uniform_u64_ptr words = (uniform_u64_ptr)(uintptr_t)L.table;     // 6 words per record
    int lo = 0, hi = L.njobs - 1;
    if (L.wgs_per_job > 0) {
        lo = wg / L.wgs_per_job;
    } else {
        while (lo < hi) {
            const int mid = (lo + hi + 1) >> 1;
            if ((int)(uint32_t)words[6 * mid + 5] <= wg) lo = mid; else hi = mid - 1;
        }
    }
    const uniform_u64_ptr rec = words + 6 * lo;
    Fp4Job job;
    job.packed = (const uint8_t *)rec[0];
    job.scales = (const uint8_t *)rec[1];
    job.x = (const float *)rec[2];
    job.y = (float *)rec[3];
    job.weight_global_scale = __uint_as_float((uint32_t)rec[4]);
    job.rows = (int)(rec[4] >> 32);
    job.tile0 = (int)(uint32_t)rec[5];
    job.x_stride = (int)(rec[5] >> 32);
    return job;
}

// T tokens per pass (1..4), WAVES waves per workgroup, STAGES steps of LDS per wave, MD dwords of block scales per
// lane (one dword = the four blocks of a 64-column group).  L.ksplit waves share a block of 32 rows, each walking
// its part of the steps; a workgroup owns WAVES / ksplit blocks of one job.
template <int T, int WAVES, int STAGES, int MD>
__global__ __launch_bounds__(WAVES * 64) void fp4_dot_kernel(const Fp4DotLaunch L) {
    static_assert(T >= 1 && T <= 4 && STAGES >= 2 && STAGES <= 4 && (MD == 16 || MD == 32), "shape");
    constexpr int WAVE_LDS = STAGES * STEP_LDS;
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    constexpr int THREADS = WAVES * 64;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const Fp4Job job = fp4_dot_find_job(L, blockIdx.x);

    const int C = L.cols;
    const int ngrp = C >> 6;                         // 64-column groups: 32 bytes of codes, four block scales
    const int nstage = dot_steps(ngrp);
    const int SG = nstage * STAGE_GROUPS;            // groups per strip (strip 1 holds the remaining ngrp - SG)
    const uint32_t row_bytes = (uint32_t)C >> 1;
    const int whole_steps = (ngrp - SG) / STAGE_GROUPS;
    const int ksplit = L.ksplit;
    const int blocks_per_wg = WAVES / ksplit;
    const int my_block = wave / ksplit, my_part = wave - my_block * ksplit;
    const int step_lo = my_part * nstage / ksplit, step_hi = (my_part + 1) * nstage / ksplit;
    // the lane's window of block scales: meta_groups groups (dwords) of its row, starting at its strip's first group
    // of the wave's steps, moved left where it would pass the row's end
    const int meta_groups = MD < (ngrp & ~3) ? MD : ngrp & ~3;
    const int want0 = step_lo * STAGE_GROUPS, want1 = SG + step_lo * STAGE_GROUPS;
    const int window0 = want0 <= ngrp - meta_groups ? want0 : ngrp - meta_groups;
    const int window1 = want1 <= ngrp - meta_groups ? want1 : ngrp - meta_groups;
    const int shift0 = want0 - window0, shift1 = want1 - window1;

    const int units = 4 * SG;                        // 32-column units per token in the image (both strips, padded)
    uint8_t *const w_lds = lds;                                            // [WAVES][STAGES][STEP_LDS]
    uint8_t *const zero_lds = lds + WAVES * WAVE_LDS;                      // FP4_ZERO_BYTES
    uint8_t *const img_lds = zero_lds + FP4_ZERO_BYTES;                    // [T][units][2 blocks][16]
    float *const xs_lds = (float *)(img_lds + (size_t)T * units * 32);     // [T][2 * units]: block scale / g
    int *const bad_lds = (int *)(xs_lds + (size_t)T * 2 * units);

    const int row_base = (((int)blockIdx.x - job.tile0) * blocks_per_wg + my_block) * BLOCK_ROWS;
    const bool has_rows = my_block < blocks_per_wg && row_base < job.rows;
    const int rows_here = !has_rows ? 1 : (job.rows - row_base < BLOCK_ROWS ? job.rows - row_base : BLOCK_ROWS);
    const int total_steps = has_rows ? step_hi - step_lo : 0;

    // ---------------------------------------------------------------- per-lane geometry (as in q4_dot.hip)
    uint8_t *const my_lds = w_lds + (size_t)wave * WAVE_LDS;
    int src_rowi[8];
    uint32_t src_col[8], src_off[8];
#pragma unroll
    for (int k = 0; k < 8; ++k) {
        const int strip = k >> 2;
        const int row = (k & 3) * 8 + (lane >> 3);
        const int piece = strip * 32 + row;
        const int seg = (lane & 7) ^ swizzle(piece);
        src_rowi[k] = row;
        src_col[k] = (uint32_t)(strip * SG) * 32u + (uint32_t)seg * 16u;
        src_off[k] = (uint32_t)row * row_bytes + src_col[k];
    }
    const int n = lane & 31, h = lane >> 5;
    const int my_piece = h * 32 + n;
    uint32_t rd_off[8];
#pragma unroll
    for (int s = 0; s < 8; ++s) rd_off[s] = (uint32_t)my_piece * 128u + (uint32_t)(s ^ swizzle(my_piece)) * 16u;
    // activation codes: row m = l % 32 of the M side is (token m / 8, strip (m / 4) % 2, block m % 4 of the unit, 0 or
    // 1); it carries codes only in the lanes of its own strip (l / 32)
    const int m_tok = n >> 3, m_strip = (n >> 2) & 1, m_block = n & 3;
    const bool has_codes = m_tok < T && m_block < 2 && m_strip == h;
    const uint8_t *const a_base = has_codes
        ? img_lds + ((size_t)(m_tok * units + 2 * m_strip * SG) * 2 + m_block) * 16
        : zero_lds;
    const uint32_t a_step = has_codes ? 2 * STAGE_GROUPS * 32 : 0u;        // eight units per step
    const uint32_t a_unit = has_codes ? 32u : 0u;
    const float *const xs_ptr = xs_lds + 4 * (h * SG);                     // the strip's first block

    // ---------------------------------------------------------------- loads
    typedef uint32_t MetaVec __attribute__((ext_vector_type(MD)));
    MetaRegs<MD> scales_r;
    MetaVec scales_v;
    auto issue_meta = [&]() {
        const int row = n < rows_here ? n : rows_here - 1;
        const size_t at = ((size_t)(row_base + row) * ngrp + (h ? window1 : window0)) * 4;
#pragma unroll
        for (int q = 0; q < MD / 4; ++q) {
            const int piece = 4 * q < meta_groups ? q : (meta_groups - 1) / 4;
            scales_r.q[q] = load_meta16(job.scales + at + 16 * piece);
        }
    };
    const uint8_t *const block_vals = job.packed + (size_t)row_base * row_bytes;
    auto issue_step = [&](int st, int slot) {
        uint8_t *const stage = my_lds + slot * STEP_LDS;
        const uint32_t advance = (uint32_t)st * (STAGE_GROUPS * 32);
        if (rows_here == BLOCK_ROWS && st < whole_steps) {
#pragma unroll
            for (int k = 0; k < 8; ++k)
                __builtin_amdgcn_global_load_lds((global_u128_ptr)(uintptr_t)(block_vals + advance + src_off[k]),
                                                 (lds_void_ptr)(stage + k * 1024), 16, 0, STREAMING);
        } else {
#pragma unroll
            for (int k = 0; k < 8; ++k) {
                const int row = src_rowi[k] < rows_here ? src_rowi[k] : rows_here - 1;
                uint32_t col = src_col[k] + advance;
                col = col <= row_bytes - 16 ? col : row_bytes - 16;
                __builtin_amdgcn_global_load_lds((global_u128_ptr)(uintptr_t)(block_vals + ((uint32_t)row * row_bytes + col)),
                                                 (lds_void_ptr)(stage + k * 1024), 16, 0, STREAMING);
            }
        }
    };

    // ---------------------------------------------------------------- arithmetic of one step
    float acc[T];
#pragma unroll
    for (int t = 0; t < T; ++t) acc[t] = 0.0f;
    const float wg = job.weight_global_scale;

    struct StepWeights { u32x4 unit[8]; };
    auto fetch = [&](int slot, StepWeights &w) {
        const uint8_t *stage = my_lds + slot * STEP_LDS;
#pragma unroll
        for (int j = 0; j < 8; ++j) w.unit[j] = *(const u32x4 *)(stage + rd_off[j]);
    };
    auto consume = [&](int st, const StepWeights &w) {
        const uint8_t *a_ptr = a_base + (uint32_t)st * a_step;
        // the step's sixteen block scales: four dwords out of the lane's registers, at a wave-uniform index for
        // either strip (blocks past the row's end meet zero codes; they take whatever the clamped index yields)
        uint32_t sc[4];
        {
            // past the registers' end (a step that straddles the row's end: its real blocks are in the last dwords,
            // the rest meet zero codes) each index is held back on its own
            const int at0 = 4 * (st - step_lo) + shift0, at1 = 4 * (st - step_lo) + shift1;
#pragma unroll
            for (int d = 0; d < 4; ++d) sc[d] = scales_v[at0 + d < MD - 1 ? at0 + d : MD - 1];
            if (at1 != at0) {                      // uniform
#pragma unroll
                for (int d = 0; d < 4; ++d) {
                    const uint32_t other = scales_v[at1 + d < MD - 1 ? at1 + d : MD - 1];
                    sc[d] = h ? other : sc[d];
                }
            }
        }
        // block scale / g of the step's sixteen blocks, per token (native vector reads: see q4_dot.hip)
        float xs[T][16];
#pragma unroll
        for (int t = 0; t < T; ++t)
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const f32x4 v = *(const f32x4 *)(xs_ptr + (size_t)t * 2 * units + st * 16 + 4 * q);
                xs[t][4 * q] = v.x; xs[t][4 * q + 1] = v.y; xs[t][4 * q + 2] = v.z; xs[t][4 * q + 3] = v.w;
            }
        // four units at a time: consecutive matrix instructions write different accumulators
#pragma unroll
        for (int half = 0; half < 2; ++half) {
            v16f d[4];
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const int j = 4 * half + k;
                const u32x4 codes = *(const u32x4 *)(a_ptr + j * a_unit);
                const v8i a = {(int)codes.x, (int)codes.y, (int)codes.z, (int)codes.w, 0, 0, 0, 0};
                const v8i b = {(int)w.unit[j].x, (int)w.unit[j].y, (int)w.unit[j].z, (int)w.unit[j].w, 0, 0, 0, 0};
                v16f zero;
#pragma unroll
                for (int i = 0; i < 16; ++i) zero[i] = 0.0f;
                d[k] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a, b, zero, 4, 4, 0, 0, 0, 0);
            }
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const int j = 4 * half + k;
                const uint32_t word = sc[j >> 1];
                // decode of the scale byte; scaled = fl(e4m3 * wg) as the reference forms it (nvfp4.c:173-192)
                const float s0 = (j & 1) ? __builtin_amdgcn_cvt_f32_fp8((int)word, 2) : __builtin_amdgcn_cvt_f32_fp8((int)word, 0);
                const float s1 = (j & 1) ? __builtin_amdgcn_cvt_f32_fp8((int)word, 3) : __builtin_amdgcn_cvt_f32_fp8((int)word, 1);
                const float scaled0 = s0 * wg, scaled1 = s1 * wg;
#pragma unroll
                for (int t = 0; t < T; ++t) {
                    acc[t] = __builtin_fmaf(scaled0 * xs[t][2 * j], d[k][4 * t], acc[t]);
                    acc[t] = __builtin_fmaf(scaled1 * xs[t][2 * j + 1], d[k][4 * t + 1], acc[t]);
                }
            }
        }
    };

    // ---------------------------------------------------------------- activation quantisation (all waves)
    // One thread per 16-column block: the reference's group-16 quantiser with closed-form encoders.  A unit of 32
    // columns is stored twice 16 bytes: block 0's codes followed by zero codes, and zero codes followed by block 1's.
    //
    // The first FP4_HELD blocks of every thread are fetched by request_blocks() before the weight loads go out and
    // waited for there: the weights then queue behind nothing, and the quantiser runs while they are on their way.
    // (Fetched after the weights, the activations are the youngest loads in flight and waiting for them waits for the
    // weights as well.)
    constexpr int FP4_HELD = 2;
    const int items = T * 2 * units;
    float held[FP4_HELD][16];
    auto fetch_block = [&](int item, float (&v)[16]) {
        const int blk = item % (2 * units);
        const int t = item / (2 * units);
#pragma unroll
        for (int q = 0; q < 16; ++q) v[q] = 0.0f;
        if (item < items && blk * 16 < C) {
            const float4 *src = reinterpret_cast<const float4 *>(job.x + (size_t)t * job.x_stride + (size_t)blk * 16);
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const float4 f = src[q];
                v[4 * q] = f.x; v[4 * q + 1] = f.y; v[4 * q + 2] = f.z; v[4 * q + 3] = f.w;
            }
        }
    };
    auto request_blocks = [&]() {
#pragma unroll
        for (int k = 0; k < FP4_HELD; ++k) fetch_block(tid + k * THREADS, held[k]);
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    };
    auto store_block = [&](int item, const float (&v)[16]) {
        const int blk = item % (2 * units);
        const int t = item / (2 * units);
        uint32_t codes[2] = {0u, 0u};
        float from_code = 0.0f;
        if (blk * 16 < C && !fp4_quantise_block(v, L.input_global_scale, codes, from_code)) *bad_lds = 1;
        uint32_t *slot = (uint32_t *)(img_lds + ((size_t)(t * units + (blk >> 1)) * 2 + (blk & 1)) * 16);
        const bool second = blk & 1;
        slot[0] = second ? 0u : codes[0]; slot[1] = second ? 0u : codes[1];
        slot[2] = second ? codes[0] : 0u; slot[3] = second ? codes[1] : 0u;
        xs_lds[(size_t)t * 2 * units + blk] = from_code;
    };
    auto build_image = [&]() {
        for (int i = tid; i < FP4_ZERO_BYTES / 4; i += THREADS) ((uint32_t *)zero_lds)[i] = 0u;
        if (tid == 0) *bad_lds = 0;
        __syncthreads();
#pragma unroll
        for (int k = 0; k < FP4_HELD; ++k)
            if (tid + k * THREADS < items) store_block(tid + k * THREADS, held[k]);
        for (int item = tid + FP4_HELD * THREADS; item < items; item += THREADS) {
            float v[16];
            fetch_block(item, v);
            store_block(item, v);
        }
    };

    auto finish_block = [&](bool bad) {
        float sum[T];
#pragma unroll
        for (int t = 0; t < T; ++t) sum[t] = acc[t] + __shfl_xor(acc[t], 32, 64);
        if (ksplit > 1) {
            float *mine = (float *)my_lds;
            asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
#pragma unroll
            for (int t = 0; t < T; ++t)
                if (lane < 32) mine[t * 32 + lane] = sum[t];
            __syncthreads();
            if (my_part != 0) return;
#pragma unroll
            for (int t = 0; t < T; ++t) {
                float total = 0.0f;
                for (int p = 0; p < ksplit; ++p)
                    total = total + ((const float *)(w_lds + (size_t)(my_block * ksplit + p) * WAVE_LDS))[t * 32 + (lane & 31)];
                sum[t] = total;
            }
        }
        if (has_rows && !bad && lane < rows_here) {
#pragma unroll
            for (int t = 0; t < T; ++t) job.y[(size_t)t * job.rows + row_base + lane] = sum[t];
        }
    };

    // ---------------------------------------------------------------- main loop (as in q4_dot.hip)
    const int first_step = total_steps > 0 ? (int)(((unsigned)blockIdx.x * WAVES + wave) % (unsigned)total_steps) : 0;
    auto step_of = [&](int g) { const int st = g + first_step; return step_lo + (st < total_steps ? st : st - total_steps); };
    request_blocks();
    if (has_rows) {
        issue_meta();
#pragma unroll
        for (int g = 0; g < STAGES; ++g)
            if (g < total_steps) issue_step(step_of(g), g);
    }
    build_image();
    __syncthreads();
    const bool bad = *bad_lds != 0;                  // uniform over the workgroup
    if (bad && tid == 0 && L.status) *L.status = -1;
    if (has_rows) {
#pragma unroll
        for (int q = 0; q < MD / 4; ++q) {
            wait_meta(scales_r.q[q]);
#pragma unroll
            for (int e = 0; e < 4; ++e) scales_v[4 * q + e] = scales_r.q[q][e];
        }
        for (int base = 0; base < total_steps; base += STAGES) {
            const bool more = static_steps(std::make_integer_sequence<int, STAGES>{}, [&](auto step_in_turn) {
                constexpr int r = decltype(step_in_turn)::value;
                const int g = base + r;
                if (g >= total_steps) return false;
                const int behind = total_steps - 1 - g < STAGES - 1 ? total_steps - 1 - g : STAGES - 1;
                if (behind == 0) wait_vm<0>();
                else if (behind == 1) wait_vm<LOADS_PER_STEP>();
                else if (behind == 2) wait_vm<2 * LOADS_PER_STEP>();
                else wait_vm<3 * LOADS_PER_STEP>();
                StepWeights w;
                fetch(r, w);
                asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
                if (g + STAGES < total_steps) issue_step(step_of(g + STAGES), r);
                consume(step_of(g), w);
                return true;
            });
            if (!more) break;
        }
    }
    finish_block(bad);
}

size_t fp4_dot_lds_bytes(int cols, int tokens, int waves, int stages) {
    const int units = 4 * dot_steps(cols >> 6) * STAGE_GROUPS;
    return (size_t)waves * stages * STEP_LDS + FP4_ZERO_BYTES + (size_t)tokens * units * (32 + 8) + 16;
}

template <int T, int WAVES, int STAGES, int MD>
int launch_shape(const Fp4DotLaunch &L, hipStream_t stream) {
    const size_t lds = fp4_dot_lds_bytes(L.cols, T, WAVES, STAGES);
    static size_t raised = 0;
    if (lds > raised) {
        if (hipFuncSetAttribute((const void *)fp4_dot_kernel<T, WAVES, STAGES, MD>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                (int)lds) != hipSuccess)
            return -1;
        raised = lds;
    }
    note_kernel("fp4_dot_kernel<%d,%d,%d,%d>", T, WAVES, STAGES, MD);
    hipLaunchKernelGGL((fp4_dot_kernel<T, WAVES, STAGES, MD>), dim3(L.total_wgs), dim3(WAVES * 64), lds, stream, L);
    return hipGetLastError() == hipSuccess ? 0 : -1;
}

}  // namespace

bool fp4_dot_takes(int cols) { return cols >= DOT_MIN_COLS && cols <= DOT_MAX_COLS && (cols & 63) == 0; }

DotShape fp4_dot_shape(int cols, int tokens, long long total_blocks) {
    const int nstage = dot_steps(cols >> 6);
    int ksplit = 1;
    while (ksplit < 8 && total_blocks * ksplit < 1024 && nstage >= 2 * ksplit) ksplit *= 2;
    // a lane's registers hold the block scales of at most 32 groups of its strip
    while ((nstage + ksplit - 1) / ksplit * STAGE_GROUPS > 32) ksplit *= 2;
    while (ksplit > 1 && ksplit > nstage) ksplit /= 2;
    // the activation codes are small: two workgroups of four waves fit every supported column count
    if (ksplit <= 4 && 2 * fp4_dot_lds_bytes(cols, tokens, 4, 2) <= DOT_LDS_LIMIT) return DotShape{4, 2, ksplit, 1};
    if (fp4_dot_lds_bytes(cols, tokens, 8, 2) <= DOT_LDS_LIMIT) return DotShape{8, 2, ksplit, 1};
    return DotShape{4, 2, ksplit <= 4 ? ksplit : 4, 1};
}

int fp4_dot_launch(const Fp4DotLaunch &launch, const DotShape &shape, hipStream_t stream) {
    Fp4DotLaunch L = launch;
    if (L.total_wgs < 1 || L.tokens < 1 || L.tokens > 4 || !fp4_dot_takes(L.cols)) return -1;
    if (shape.ksplit < 1 || shape.waves % shape.ksplit) return -1;
    if (fp4_dot_lds_bytes(L.cols, L.tokens, shape.waves, shape.stages) > DOT_LDS_LIMIT) return -1;
    L.ksplit = shape.ksplit;
    const int groups = (dot_steps(L.cols >> 6) + shape.ksplit - 1) / shape.ksplit * STAGE_GROUPS;
    if (groups > 32) return -1;
    const int md = groups <= 16 ? 16 : 32;
#define FP4_DOT_CASE(TT, WW) \
    if (L.tokens == TT && shape.waves == WW && shape.stages == 2) \
        return md == 16 ? launch_shape<TT, WW, 2, 16>(L, stream) : launch_shape<TT, WW, 2, 32>(L, stream)
    FP4_DOT_CASE(1, 4); FP4_DOT_CASE(2, 4); FP4_DOT_CASE(3, 4); FP4_DOT_CASE(4, 4);
    FP4_DOT_CASE(1, 8); FP4_DOT_CASE(2, 8); FP4_DOT_CASE(3, 8); FP4_DOT_CASE(4, 8);
#undef FP4_DOT_CASE
    return -1;
}

}  // namespace mi355
