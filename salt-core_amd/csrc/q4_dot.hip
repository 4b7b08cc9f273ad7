// Affine-Q4 matvec for gfx950, tolerance class: the HBM-bound decode kernel.
//
// The reference row (src/kernels.c:220-250) rounds every weight, product and sum and fixes the order of 32 chains;
// reproducing that costs about four vector instructions per weight, which caps a bit-exact kernel below the memory
// system.  This kernel computes the same sum in a different association, per 64-column scale group g of a row:
//
//     y = sum_g ( scale_g * sum_{c in g} q_c * x_c  +  bias_g * sum_{c in g} x_c )
//
// and evaluates the inner integer-by-activation dot products exactly:
//  * each activation group is turned into block fixed point once per workgroup: I_c = rint(x_c * 2^k_g) with k_g
//    chosen so that |I_c| < 2^30, split into four signed 8-bit digit planes  I = d0 + 2^8 d1 + 2^16 d2 + 2^24 d3.
//    The error of x against its fixed-point image is at most 2^-31 of the group's largest magnitude.
//  * the codes q (0..15) are 8-bit integers after two masks and a shift, so  sum_c q_c * d_p,c  is an integer dot
//    product: v_mfma_i32_32x32x32_i8 computes it for 32 rows at a time.  The matrix instruction is used as a bank
//    of dot-product units: its N side holds 32 weight rows, its M side the digit planes of up to four tokens, its K
//    side sixteen columns of each of two groups.  Digit planes of the "other" group are zero, which keeps the two
//    groups' sums apart in different output rows.
//  * the four plane sums (each below 2^17) are recombined in integers and converted to fp32 once per group; the
//    group's scale, its power of two and the bias term follow as two fused multiply-adds per (row, group, token).
//    sum_c x_c of a group is accumulated in double and rounded once.
// Everything except the last two steps is exact, so the result differs from the infinitely precise sum by a few
// fp32 roundings per group.  Stated bound (tests): |y - y_ref| <= 2^-20 * sum_c (|q_c s| + 16|s| + |b|) |x_c| + 1e-6.
//
// Data movement: a wave owns blocks of 32 rows and walks each in two strips (halves of the row) at once, 128 bytes
// of each strip and row per step: 8 KiB per step, fetched straight into LDS with eight 16-byte-per-lane loads
// (contiguous 128-byte pieces in memory, non-temporal).  Several steps are in flight per wave and there is no
// barrier after the prologue.  Lane (row n, strip h) reads its
// 32 bytes of a group back with two 16-byte LDS reads (slots swizzled by the row so that the lanes of a read phase
// hit different bank groups).  The scales and biases of a block do not travel with the steps: a lane fetches the
// scales and biases of its row and strip for the whole block into registers before the stream starts, and picks
// the step's four by register indexing.  (Fetching them per step with direct-to-LDS loads of 16 bytes per lane
// costs a quarter of the stream's rate: 64 scattered pieces per load.  Loads that return to registers are kept out
// of the loop on purpose: on this device they do not complete in issue order with direct-to-LDS loads, so a partial
// s_waitcnt vmcnt(n) cannot tell which of the two kinds has landed.)
#include "dot_common.h"
#include "q4_image.h"
#include "device_math.h"
#include "router_device.h"

#include <stdio.h>
#include <string.h>

namespace mi355 {
namespace {

__device__ __forceinline__ Q4Job dot_find_job(const Q4DotLaunch &L, int wg) {
    if (L.table == nullptr && L.njobs <= 1) return L.one;
    // 7 words per record, in a device table or inside the kernel arguments (the launch record is the kernel's only
    // argument, so the inline records sit at their offset in the kernarg segment)
    const uniform_u64_ptr words =
        L.table ? (uniform_u64_ptr)(uintptr_t)L.table
                : (uniform_u64_ptr)((const char __attribute__((address_space(4))) *)__builtin_amdgcn_kernarg_segment_ptr() +
                                    offsetof(Q4DotLaunch, inline_jobs));
    int lo = 0, hi = L.njobs - 1;
    if (L.wgs_per_job > 0) {               // every job has the same number of workgroups: no search
        lo = wg / L.wgs_per_job;
    } else {
        while (lo < hi) {                  // last job whose first workgroup is <= wg
            const int mid = (lo + hi + 1) >> 1;
            if ((int)(words[7 * mid + 5] >> 32) <= wg) lo = mid; else hi = mid - 1;
        }
    }
    const uniform_u64_ptr rec = words + 7 * lo;
    Q4Job job;
    job.vals = (const uint8_t *)rec[0];
    job.scales = (const uint8_t *)rec[1];
    job.biases = (const uint8_t *)rec[2];
    job.x = (const float *)rec[3];
    job.y = (float *)rec[4];
    job.rows = (int)(uint32_t)rec[5];
    job.tile0 = (int)(rec[5] >> 32);
    job.x_stride = (int)(uint32_t)rec[6];
    job.y_stride = (int)(rec[6] >> 32);
    return job;
}

// T tokens per pass (1..4), WAVES waves per workgroup, STAGES steps of LDS per wave (one being consumed, the others
// in flight), MD dwords of scales per lane (two groups each: 16 serves rows of up to 4096 columns, 32 up to 8192).
// A workgroup owns WAVES consecutive blocks of 32 rows of one job, one per wave.
//
// PRO selects a prologue of the MoE decode step (0: none, the jobs come from the launch): 1 = router top-k, the
// workgroup derives its gate or up job from the selection (one workgroup past the jobs publishes selection, weights
// and status); 2 = the down projection of one selected expert, whose activation gelu_tanh(gate) * up is computed
// while the digit planes are built.
template <int T, int WAVES, int STAGES, int MD, int PRO = 0>
__global__ __launch_bounds__(WAVES * 64) void q4_dot_kernel(const Q4DotLaunch L) {
    constexpr int NB = 1;        // blocks of 32 rows a wave walks back to back (launches with many blocks take the
                                 // sixteen-row kernel instead of a longer walk here)
    static_assert(T >= 1 && T <= 4 && STAGES >= 2 && STAGES <= 4 && (MD == 16 || MD == 32), "tokens per pass, steps per wave");
    static_assert(PRO == 0 || (T == 1 && sizeof(RouterShared) <= (size_t)WAVES * STAGES * STEP_LDS),
                  "the MoE prologues serve one token; the router borrows the weight staging memory");
    constexpr int WAVE_LDS = STAGES * STEP_LDS;
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    constexpr int THREADS = WAVES * 64;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    Q4Job job;
    const float *act_gate = nullptr, *act_up = nullptr;       // PRO == 2: the activation is gelu_tanh(gate) * up
    if (PRO == 0) {
        job = dot_find_job(L, blockIdx.x);
    } else {
        const MoeFuse &m = L.moe;
        const size_t n = (size_t)m.hidden * (size_t)m.routed;
        const size_t vals_bytes = n / 2, meta_bytes = (n / 64) * 2, proj_bytes = vals_bytes + 2 * meta_bytes;
        const int wgs_per_job = L.wgs_per_job;
        const int slot = (int)blockIdx.x / wgs_per_job;
        if (PRO == 1) {
            // The expert, and with it the weight pointers, is known only after the router has run; everything else
            // is known now, so that the activation's digit planes can be built while the logits are on their way.
            const int place = slot >> 1, proj = slot & 1;                  // slot = 2 * place + (0 gate | 1 up)
            job.vals = nullptr;
            job.x = m.x;
            job.y = (proj ? m.up : m.gate) + (size_t)place * m.routed;
            job.rows = m.routed;
            job.x_stride = m.hidden;
            job.y_stride = m.routed;
        } else {
            if (*(const int __attribute__((address_space(4))) *)(uintptr_t)m.status != 0) return;
            const int place = slot;
            const int expert = ((const int __attribute__((address_space(4))) *)(uintptr_t)m.selected)[place];
            act_gate = m.gate + (size_t)place * m.routed;
            act_up = m.up + (size_t)place * m.routed;
            job.vals = m.pool + (size_t)expert * m.expert_stride + 2 * proj_bytes;
            job.x = nullptr;
            job.y = m.expert_out + (size_t)place * m.hidden;
            job.rows = m.hidden;
            job.x_stride = m.routed;
            job.y_stride = m.hidden;
        }
        job.tile0 = slot * wgs_per_job;
        job.scales = job.vals + vals_bytes;
        job.biases = job.scales + meta_bytes;
    }
    const bool publisher = PRO == 1 && (int)blockIdx.x == L.total_wgs;     // one workgroup past the jobs

    const int C = L.cols;
    const int ngrp = C >> 6;
    // Groups per strip: half the row, rounded up to whole steps so that strip 1 starts on a 128-byte boundary of the
    // row (a piece that straddles two memory lines is fetched twice by loads that bypass the caches).  Strip 1 holds
    // the remaining ngrp - SG groups.
    const int nstage = dot_steps(ngrp);
    const int SG = nstage * STAGE_GROUPS;
    const uint32_t row_bytes = (uint32_t)C >> 1;
    const int whole_steps = (ngrp - SG) / STAGE_GROUPS;            // steps that lie inside the row for both strips
    // The row may be cut into L.ksplit parts along its columns (launches with few blocks): a wave then walks only the
    // steps [step_lo, step_hi) of its block, and the parts of a block are added in order at the end.
    const int ksplit = L.ksplit;
    const int blocks_per_wg = WAVES / ksplit;
    const int my_block = wave / ksplit, my_part = wave - my_block * ksplit;
    const int step_lo = my_part * nstage / ksplit, step_hi = (my_part + 1) * nstage / ksplit;
    // A lane holds the scales (and biases) of meta_groups consecutive groups of its row in registers: a window that
    // starts at its strip's first group of the wave's steps, moved left where it would pass the row's end.
    const int meta_groups = 2 * MD < (ngrp & ~7) ? 2 * MD : ngrp & ~7;
    const int want0 = step_lo * STAGE_GROUPS, want1 = SG + step_lo * STAGE_GROUPS;
    const int window0 = want0 <= ngrp - meta_groups ? want0 : ngrp - meta_groups;
    const int window1 = want1 <= ngrp - meta_groups ? want1 : ngrp - meta_groups;
    const int shift0 = want0 - window0, shift1 = want1 - window1;  // groups between the window's start and the first step's

    uint8_t *const w_lds = lds;                                            // [WAVES][STAGES][STEP_LDS]
    uint8_t *const zero_lds = lds + WAVES * WAVE_LDS;                      // ZERO_BYTES
    uint8_t *const img_lds = zero_lds + ZERO_BYTES;                        // [T][2 * SG][GROUP_IMAGE]
    float *const xm_lds = (float *)(img_lds + (size_t)T * 2 * SG * GROUP_IMAGE);   // [T][2 * SG] (power of two, sum)

    // the wave's blocks and its stream of steps
    const int row_base0 = (((int)blockIdx.x - job.tile0) * blocks_per_wg + my_block) * (NB * BLOCK_ROWS);
    auto row_base_of = [&](int b) { return row_base0 + b * BLOCK_ROWS; };
    auto rows_of = [&](int b) {                       // 1..32; a block past the job's rows is never walked
        const int left = job.rows - row_base_of(b);
        return left < 1 ? 1 : (left < BLOCK_ROWS ? left : BLOCK_ROWS);
    };
    int live_blocks = 0;                             // a wave without rows still helps with the activations
#pragma unroll
    for (int b = 0; b < NB; ++b) live_blocks += my_block < blocks_per_wg && row_base_of(b) < job.rows;
    const bool has_rows = live_blocks > 0;
    const int steps_per_block = step_hi - step_lo;
    const int total_steps = live_blocks * steps_per_block;

    // ---------------------------------------------------------------- per-lane geometry
    // weights: load k of a step covers strip k / 4, rows 8 (k % 4) .. + 7 of the block; lane i lands in slot 64 k + i,
    // that is piece (strip * 32 + row), position i % 8, which receives segment (i % 8) ^ swizzle(piece) of the piece
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
    // reads: lane (n, h) owns piece h * 32 + n
    const int n = lane & 31, h = lane >> 5;
    const int my_piece = h * 32 + n;
    uint32_t rd_off[8];
#pragma unroll
    for (int s = 0; s < 8; ++s) rd_off[s] = (uint32_t)my_piece * 128u + (uint32_t)(s ^ swizzle(my_piece)) * 16u;
    // a job without biases: the load still happens (the waits count it, it reads the scales); its result is dropped
    const bool no_bias = PRO == 0 && job.biases == nullptr;
    // digit planes: row m = l % 32 of the M side is (token m / 8, strip (m / 4) % 2, plane m % 4); it carries digits
    // only in the lanes of its own strip (l / 32)
    const int m_tok = n >> 3, m_strip = (n >> 2) & 1, m_plane = n & 3;
    const bool has_digits = m_tok < T && m_strip == h;
    const uint8_t *const a_base = has_digits
        ? img_lds + ((size_t)(m_tok * 2 * SG + m_strip * SG) * 16 + m_plane) * 16
        : zero_lds + 64;              // a bank group that no digit plane of the same read occupies
    const uint32_t a_step = has_digits ? STAGE_GROUPS * GROUP_IMAGE : 0u;
    const float *const xm_ptr = xm_lds + 2 * (h * SG);

    // ---------------------------------------------------------------- loads
    // The block's scales and biases: lane (n, h) fetches 2 * MD groups of row n, 16 bytes at a time.
    typedef uint32_t MetaVec __attribute__((ext_vector_type(MD * NB)));
    MetaRegs<MD> scales_r[NB], biases_r[NB];
    MetaVec scales_v, biases_v;                      // the same registers as one indexable vector, valid after the wait
    auto issue_meta = [&](int b) {
        const int rows_here = rows_of(b);
        const int row = n < rows_here ? n : rows_here - 1;
        const size_t at = ((size_t)(row_base_of(b) + row) * ngrp + (h ? window1 : window0)) * 2;
#pragma unroll
        for (int q = 0; q < MD / 4; ++q) {
            // pieces past the window are not fetched (and never read): the address repeats the last real one
            const int piece = 8 * q < meta_groups ? q : (meta_groups - 1) / 8;
            scales_r[b].q[q] = load_meta16(job.scales + at + 16 * piece);
            biases_r[b].q[q] = load_meta16((no_bias ? job.scales : job.biases) + at + 16 * piece);
        }
    };
    // Step st of the wave's block b into ring slot `slot`: eight weight pieces.
    auto issue_step = [&](int b, int st, int slot) {
        const int rows_here = rows_of(b);
        const uint8_t *const block_vals = job.vals + (size_t)row_base_of(b) * row_bytes;
        uint8_t *const stage = my_lds + slot * STEP_LDS;
        const uint32_t advance = (uint32_t)st * (STAGE_GROUPS * 32);
        if (rows_here == BLOCK_ROWS && st < whole_steps) {
            // a wave-uniform base that advances with the step plus a fixed 32-bit offset per lane
#pragma unroll
            for (int k = 0; k < 8; ++k)
                __builtin_amdgcn_global_load_lds((global_u128_ptr)(uintptr_t)(block_vals + advance + src_off[k]),
                                                 (lds_void_ptr)(stage + k * 1024), 16, 0, STREAMING);
        } else {
            // the matrix ends inside this block, or strip 1 ends inside this step or before it: stay inside
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
    // A step's weights leave LDS for registers in one go: its slot is then free for the loads of a later step while
    // the arithmetic runs.
    struct StepWeights { uint32_t raw[STAGE_GROUPS][8]; };
    auto fetch = [&](int slot, StepWeights &w) {
        const uint8_t *stage = my_lds + slot * STEP_LDS;
#pragma unroll
        for (int u = 0; u < STAGE_GROUPS; ++u) {
            const u32x4 w0 = *(const u32x4 *)(stage + rd_off[2 * u]);
            const u32x4 w1 = *(const u32x4 *)(stage + rd_off[2 * u + 1]);
            w.raw[u][0] = w0.x; w.raw[u][1] = w0.y; w.raw[u][2] = w0.z; w.raw[u][3] = w0.w;
            w.raw[u][4] = w1.x; w.raw[u][5] = w1.y; w.raw[u][6] = w1.z; w.raw[u][7] = w1.w;
        }
    };
    auto consume = [&](int b, int st, const StepWeights &w) {
        const uint8_t *a_ptr = a_base + (uint32_t)st * a_step;
        // the step's four scales and four biases: two dwords each out of the lane's registers, at a wave-uniform
        // index for either strip (groups past the row's end have zero digits; they take whatever the clamped index
        // yields, a finite value of the row)
        float scale[STAGE_GROUPS], bias[STAGE_GROUPS];
        {
            // register indexing by a wave-uniform index
            auto pick = [&](const MetaVec &m, int dword) -> uint32_t { return m[dword]; };
            // A step's four groups are two dwords; past the registers' end (a step that straddles the row's end: its
            // real groups are in the last dword, the rest meet zero digits) each index is held back on its own
            const int at0 = 2 * (st - step_lo) + (shift0 >> 1), at1 = 2 * (st - step_lo) + (shift1 >> 1);
            const int lo0 = b * MD + (at0 < MD - 1 ? at0 : MD - 1), hi0 = b * MD + (at0 + 1 < MD - 1 ? at0 + 1 : MD - 1);
            const int lo1 = b * MD + (at1 < MD - 1 ? at1 : MD - 1), hi1 = b * MD + (at1 + 1 < MD - 1 ? at1 + 1 : MD - 1);
            uint32_t s_lo = pick(scales_v, lo0), s_hi = pick(scales_v, hi0);
            uint32_t b_lo = pick(biases_v, lo0), b_hi = pick(biases_v, hi0);
            if (at1 != at0) {                      // uniform
                const uint32_t s_lo1 = pick(scales_v, lo1), s_hi1 = pick(scales_v, hi1);
                const uint32_t b_lo1 = pick(biases_v, lo1), b_hi1 = pick(biases_v, hi1);
                s_lo = h ? s_lo1 : s_lo; s_hi = h ? s_hi1 : s_hi;
                b_lo = h ? b_lo1 : b_lo; b_hi = h ? b_hi1 : b_hi;
            }
            scale[0] = __uint_as_float(s_lo << 16); scale[1] = __uint_as_float(s_lo & 0xffff0000u);
            scale[2] = __uint_as_float(s_hi << 16); scale[3] = __uint_as_float(s_hi & 0xffff0000u);
            bias[0] = __uint_as_float(b_lo << 16); bias[1] = __uint_as_float(b_lo & 0xffff0000u);
            bias[2] = __uint_as_float(b_hi << 16); bias[3] = __uint_as_float(b_hi & 0xffff0000u);
        }
        // (power of two, sum) of the step's four groups, per token.  Read as native vectors: an LDS read without type
        // information (a struct such as float4, or reads the compiler merged itself) is made to wait for every
        // outstanding direct-to-LDS load
        float xm[T][2 * STAGE_GROUPS];
#pragma unroll
        for (int t = 0; t < T; ++t) {
            const f32x4 lo4 = *(const f32x4 *)(xm_ptr + 2 * (t * 2 * SG + st * STAGE_GROUPS));
            const f32x4 hi4 = *(const f32x4 *)(xm_ptr + 2 * (t * 2 * SG + st * STAGE_GROUPS) + 4);
            xm[t][0] = lo4.x; xm[t][1] = lo4.y; xm[t][2] = lo4.z; xm[t][3] = lo4.w;
            xm[t][4] = hi4.x; xm[t][5] = hi4.y; xm[t][6] = hi4.z; xm[t][7] = hi4.w;
        }
        // The four groups advance together through the four quarters, so that consecutive matrix instructions belong
        // to different accumulators and never wait for each other.
        v16i d[STAGE_GROUPS];
#pragma unroll
        for (int u = 0; u < STAGE_GROUPS; ++u)
#pragma unroll
            for (int i = 0; i < 16; ++i) d[u][i] = 0;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            v4i a[STAGE_GROUPS];
#pragma unroll
            for (int u = 0; u < STAGE_GROUPS; ++u) a[u] = *(const v4i *)(a_ptr + u * GROUP_IMAGE + j * 64);
#pragma unroll
            for (int u = 0; u < STAGE_GROUPS; ++u) {
                const uint32_t lo = w.raw[u][2 * j], hi = w.raw[u][2 * j + 1];
                v4i b;
                b.x = (int)(lo & 0x0f0f0f0fu);
                b.y = (int)((lo >> 4) & 0x0f0f0f0fu);
                b.z = (int)(hi & 0x0f0f0f0fu);
                b.w = (int)((hi >> 4) & 0x0f0f0f0fu);
                d[u] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[u], b, d[u], 0, 0, 0);
            }
        }
#pragma unroll
        for (int u = 0; u < STAGE_GROUPS; ++u) {
            const float bias_u = no_bias ? 0.0f : bias[u];
#pragma unroll
            for (int t = 0; t < T; ++t) {
                const int lo = d[u][4 * t] + (d[u][4 * t + 1] << 8);
                const int hi = d[u][4 * t + 2] + (d[u][4 * t + 3] << 8);
                const float f = __builtin_fmaf((float)hi, 65536.0f, (float)lo);
                acc[t] = __builtin_fmaf(scale[u] * xm[t][2 * u], f, acc[t]);
                acc[t] = __builtin_fmaf(bias_u, xm[t][2 * u + 1], acc[t]);
            }
        }
    };

    // The two strips of a row meet; with the row cut into parts, every wave leaves its sums in its own (now idle)
    // LDS and the first wave of the block adds them in part order.
    auto finish_block = [&](int b) {
        const int row_base = row_base_of(b), rows_here = rows_of(b);
        const bool block_has_rows = my_block < blocks_per_wg && row_base < job.rows;
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
        if (block_has_rows && lane < rows_here) {
#pragma unroll
            for (int t = 0; t < T; ++t) job.y[(size_t)t * job.y_stride + row_base + lane] = sum[t];
        }
#pragma unroll
        for (int t = 0; t < T; ++t) acc[t] = 0.0f;
    };

    // ---------------------------------------------------------------- activations -> digit planes (all waves)
    auto build_image = [&]() {
        build_q4_image<T, THREADS>(tid, ngrp, SG, zero_lds, img_lds, xm_lds, T, [&](int t, size_t column, float (&xv)[8]) {
            if (PRO == 2) {
#pragma unroll
                for (int k = 0; k < 8; ++k) xv[k] = det_gelu_tanh(act_gate[column + k]) * act_up[column + k];
            } else {
                const float *src = job.x + (size_t)t * job.x_stride + column;
#pragma unroll
                for (int k = 0; k < 8; ++k) xv[k] = src[k];
            }
        });
    };

    // ---------------------------------------------------------------- main loop
    // Weight loads go out in step order, LOADS_PER_STEP per step, STAGES steps ahead: a step's slot is refilled as
    // soon as its weights sit in registers, before its arithmetic.  When step g is waited for, what may still be in
    // flight is exactly the steps behind it: direct-to-LDS loads complete in issue order.  The first loads do not
    // depend on the activations: they are on their way while the digit planes are built.  The scales and biases, the
    // only loads that return to registers, are waited for with everything that is in flight at that moment, once.
    // Blocks start their walk over the row at different steps: rows whose length is a power of two put the same
    // step of every row on the same memory channels, and waves that all began at step 0 would queue there.
    const int first_step = steps_per_block > 0 ? (int)(((unsigned)blockIdx.x * WAVES + wave) % (unsigned)steps_per_block) : 0;
    // step g of the stream: block g / steps_per_block, and inside the block the walk that starts at first_step
    auto block_of = [&](int g) { return NB == 1 ? 0 : g / steps_per_block; };
    auto step_of = [&](int g) {
        const int st = (NB == 1 ? g : g - block_of(g) * steps_per_block) + first_step;
        return step_lo + (st < steps_per_block ? st : st - steps_per_block);
    };
    if (PRO == 1) {
        const MoeFuse &m = L.moe;
        // first touch of the router's inputs now: they arrive while the digit planes are built
        float warm = 0.0f;
        if (tid < m.n_experts) warm = m.logits[tid] + m.per_expert_scale[tid];
        if (!publisher) build_image();
        asm volatile("" ::"v"(warm));
        const int slot = (int)blockIdx.x / L.wgs_per_job;
        int expert;
        if (publisher) {
            // the workgroup that publishes selection, weights and status runs the whole router (ordered sums and all)
            RouterShared &sh = *reinterpret_cast<RouterShared *>(lds);     // the weight staging memory, idle here
            router_topk_block(m.logits, m.per_expert_scale, m.n_experts, m.topk, true, true, sh);
            const int bad = sh.bad;
            if (tid == 0) *m.status = bad ? -1 : 0;
            if (tid < m.topk && !bad) { m.selected[tid] = sh.out_sel[tid]; m.weights[tid] = sh.out_w[tid]; }
            return;
        }
        // every other wave finds its expert on its own: with finite inputs the router cannot fail later
        expert = router_select_wave(m.logits, m.per_expert_scale, m.n_experts, m.topk, slot >> 1);
        if (expert < 0) return;                                            // uniform: every wave sees the same inputs
        const size_t n_weights = (size_t)m.hidden * (size_t)m.routed;
        const size_t vals_bytes = n_weights / 2, meta_bytes = (n_weights / 64) * 2;
        job.vals = m.pool + (size_t)expert * m.expert_stride + (size_t)(slot & 1) * (vals_bytes + 2 * meta_bytes);
        job.scales = job.vals + vals_bytes;
        job.biases = job.scales + meta_bytes;
    }
    // Plain launches: the activations are sent for first and the weights when they have arrived, so that the digit
    // planes are built while the weights are on their way (weights first, activations queued behind them, cost a
    // launch of one matrix up to a microsecond).
    const ImageItems items(T, ngrp);
    Q4ImageBuilder<THREADS> image;
    if (PRO == 0) {
        image.request_early(tid, items, [&](int t) { return job.x + (size_t)t * job.x_stride; });
        image.settle(0, items);
    }
    if (has_rows) {
#pragma unroll
        for (int b = 0; b < NB; ++b)
            if (b < live_blocks) issue_meta(b);
#pragma unroll
        for (int g = 0; g < STAGES; ++g)
            if (g < total_steps) issue_step(block_of(g), step_of(g), g);
    }
    if (PRO == 0) {
        image.build(tid, items, SG, zero_lds, img_lds, xm_lds, [&](int t, size_t column, float (&xv)[8]) {
            const float *src = job.x + (size_t)t * job.x_stride + column;
#pragma unroll
            for (int k = 0; k < 8; ++k) xv[k] = src[k];
        });
    } else if (PRO != 1) {
        build_image();
    }
    __syncthreads();
    if (has_rows) {
#pragma unroll
    for (int b = 0; b < NB; ++b)
#pragma unroll
    for (int q = 0; q < MD / 4; ++q) {
        if (b >= live_blocks) { scales_r[b].q[q] = u32x4{0u, 0u, 0u, 0u}; biases_r[b].q[q] = u32x4{0u, 0u, 0u, 0u}; }
        wait_meta(scales_r[b].q[q]);
        wait_meta(biases_r[b].q[q]);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            scales_v[b * MD + 4 * q + e] = scales_r[b].q[q][e];
            biases_v[b * MD + 4 * q + e] = biases_r[b].q[q][e];
        }
    }
    if ((shift0 | shift1) & 1) {
        // a window that starts an odd number of groups before the strip's first step: move the lane's values down by
        // one group (16 bits), so that a step's four again fill two whole registers
        const bool odd = ((h ? shift1 : shift0) & 1) != 0;
#pragma unroll
        for (int i = 0; i < MD * NB; ++i) {
            const uint32_t s_next = (i + 1) % MD ? scales_v[i + 1] : 0u, b_next = (i + 1) % MD ? biases_v[i + 1] : 0u;
            const uint32_t s_moved = __builtin_amdgcn_alignbit(s_next, scales_v[i], 16);
            const uint32_t b_moved = __builtin_amdgcn_alignbit(b_next, biases_v[i], 16);
            scales_v[i] = odd ? s_moved : scales_v[i];
            biases_v[i] = odd ? b_moved : biases_v[i];
        }
    }

    for (int base = 0; base < total_steps; base += STAGES) {
        const bool more = static_steps(std::make_integer_sequence<int, STAGES>{}, [&](auto step_in_turn) {
            constexpr int r = decltype(step_in_turn)::value;       // ring slot of step base + r
            const int g = base + r;
            if (g >= total_steps) return false;
            {
                const int behind = total_steps - 1 - g < STAGES - 1 ? total_steps - 1 - g : STAGES - 1;
                if (behind == 0) wait_vm<0>();
                else if (behind == 1) wait_vm<LOADS_PER_STEP>();
                else if (behind == 2) wait_vm<2 * LOADS_PER_STEP>();
                else wait_vm<3 * LOADS_PER_STEP>();
            }
            StepWeights w;
            fetch(r, w);
            // the reads have returned before the slot is written again
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
            if (g + STAGES < total_steps) issue_step(block_of(g + STAGES), step_of(g + STAGES), r);
            consume(block_of(g), step_of(g), w);
            // the last step of a block that is not the wave's last: its rows are complete
            if (NB > 1 && (g + 1) % steps_per_block == 0 && g + 1 < total_steps) finish_block(block_of(g));
            return true;
        });
        if (!more) break;
    }
    }   // has_rows
    finish_block(live_blocks > 0 ? live_blocks - 1 : 0);
}

size_t dot_lds_bytes(int cols, int tokens, int waves, int stages) {
    const int sg = dot_steps(cols >> 6) * STAGE_GROUPS;
    return (size_t)waves * stages * STEP_LDS + ZERO_BYTES + (size_t)tokens * 2 * sg * (GROUP_IMAGE + 8);
}

template <int T, int WAVES, int STAGES, int MD, int PRO = 0>
int launch_shape(const Q4DotLaunch &L, hipStream_t stream) {
    const size_t lds = dot_lds_bytes(L.cols, T, WAVES, STAGES);
    static size_t raised = 0;                 // per instantiation: the largest dynamic LDS size asked for so far
    if (lds > raised) {
        if (hipFuncSetAttribute((const void *)q4_dot_kernel<T, WAVES, STAGES, MD, PRO>,
                                hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess)
            return -1;
        raised = lds;
    }
    note_kernel("q4_dot_kernel<%d,%d,%d,%d,%d> ksplit %d", T, WAVES, STAGES, MD, PRO, L.ksplit);
    // the router prologue has one more workgroup: the one that publishes its outputs
    hipLaunchKernelGGL((q4_dot_kernel<T, WAVES, STAGES, MD, PRO>), dim3(L.total_wgs + (PRO == 1 ? 1 : 0)),
                       dim3(WAVES * 64), lds, stream, L);
    return hipGetLastError() == hipSuccess ? 0 : -1;
}

// (waves per workgroup, steps of LDS per wave); `resident` workgroups share a compute unit's LDS.  Every entry is
// the first fit for some (columns, tokens, blocks): {4,2,2} rows of up to 3584 columns; {3,2,2} wider rows that are
// not cut; {8,2,1} rows cut in 2, 4 or 8; {7,2,1} 8192 columns uncut; {6,2,1} 8192 columns cut in 2; {4,3,1} 8192
// columns cut in 4; {4,2,1} several tokens of 8192 columns.
struct Candidate { int waves, stages, resident; };
constexpr Candidate CANDIDATES[] = {{4, 2, 2}, {3, 2, 2}, {8, 2, 1}, {7, 2, 1}, {6, 2, 1}, {4, 3, 1}, {4, 2, 1}};

}  // namespace

bool q4_dot_takes(int cols) { return cols >= DOT_MIN_COLS && cols <= DOT_MAX_COLS && (cols & 63) == 0; }

int q4_dot_tokens_per_pass(int cols) {
    // what fits beside four waves' weight steps in 160 KiB of LDS
    for (int t = 4; t >= 1; --t)
        if (dot_lds_bytes(cols, t, 4, 2) <= DOT_LDS_LIMIT) return t;
    return 0;
}

DotShape q4_dot_shape(int cols, int tokens, long long total_blocks) {
    const int nstage = dot_steps(cols >> 6);
    // Few blocks: cut the rows along their columns until the launch has about a thousand waves
    int ksplit = 1;
    while (ksplit < 8 && total_blocks * ksplit < 1024 && nstage >= 2 * ksplit) ksplit *= 2;
    while (ksplit > 1 && ksplit > nstage) ksplit /= 2;
    // in order of preference; the first that fits the LDS beside the digit planes is taken
    for (const Candidate &c : CANDIDATES)
        if (c.waves % ksplit == 0 && (ksplit == 1 || c.waves >= 4) &&
            dot_lds_bytes(cols, tokens, c.waves, c.stages) * c.resident <= DOT_LDS_LIMIT) {
            return DotShape{c.waves, c.stages, ksplit, 1};
        }
    return DotShape{4, 2, ksplit <= 4 ? ksplit : 4, 1};
}

int q4_dot_launch(const Q4DotLaunch &launch, const DotShape &shape, hipStream_t stream) {
    Q4DotLaunch L = launch;
    if (L.total_wgs < 1 || L.tokens < 1 || L.tokens > 4 || !q4_dot_takes(L.cols)) return -1;
    if (dot_lds_bytes(L.cols, L.tokens, shape.waves, shape.stages) > DOT_LDS_LIMIT) return -1;
    if (shape.ksplit < 1 || shape.waves % shape.ksplit) return -1;
    L.ksplit = shape.ksplit;
    // groups of a strip that one wave walks: its registers hold 32 (MD = 16) or 64 (MD = 32)
    const int steps = dot_steps(L.cols >> 6);
    const int md = ((steps + shape.ksplit - 1) / shape.ksplit) * STAGE_GROUPS <= 32 ? 16 : 32;
    if (shape.blocks_per_wave != 1) return -1;
#define DOT_CASE(TT, WW, SS) \
    if (L.tokens == TT && shape.waves == WW && shape.stages == SS) \
        return md == 16 ? launch_shape<TT, WW, SS, 16>(L, stream) : launch_shape<TT, WW, SS, 32>(L, stream)
#define DOT_CASES(TT) DOT_CASE(TT, 8, 2); DOT_CASE(TT, 7, 2); DOT_CASE(TT, 6, 2); DOT_CASE(TT, 4, 3); DOT_CASE(TT, 4, 2); \
                      DOT_CASE(TT, 3, 2)
    DOT_CASES(1); DOT_CASES(2); DOT_CASES(3); DOT_CASES(4);
#undef DOT_CASES
#undef DOT_CASE
    return -1;
}

// The two matvec launches of the MoE decode step on the streaming kernel: four waves per workgroup, the rows cut
// along their columns so that every compute unit gets work.  Geometries the prologues do not serve return -1 (the
// caller then takes the bit-exact plan).
static bool moe_dot_geometry_ok(const MoeFuse &m) {
    return m.n_experts >= 1 && m.n_experts <= 256 && m.topk >= 1 && m.topk <= m.n_experts && m.topk <= ROUTER_MAX_TOPK &&
           q4_dot_takes(m.hidden) && q4_dot_takes(m.routed) && m.hidden <= 4096 && m.routed <= 4096;
}

// Whether q4_dot_moe_gate_up_launch and q4_dot_moe_down_launch serve this geometry (a refusal there is then a failure).
bool q4_dot_moe_serves(const MoeFuse &m) {
    return moe_dot_geometry_ok(m) && dot_lds_bytes(m.hidden, 1, 4, 2) <= DOT_LDS_LIMIT &&
           dot_lds_bytes(m.routed, 1, 4, 2) <= DOT_LDS_LIMIT;
}

static int moe_dot_ksplit(long long blocks, int cols) {
    const int nstage = dot_steps(cols >> 6);
    int ksplit = 1;
    while (ksplit < 4 && blocks * ksplit < 1024 && nstage >= 2 * ksplit) ksplit *= 2;
    return ksplit;
}

int q4_dot_moe_gate_up_launch(const MoeFuse &m, hipStream_t stream) {
    if (!moe_dot_geometry_ok(m) || dot_lds_bytes(m.hidden, 1, 4, 2) > DOT_LDS_LIMIT) return -1;
    Q4DotLaunch L;
    memset(&L, 0, sizeof L);
    L.moe = m;
    L.cols = m.hidden; L.tokens = 1; L.njobs = 2 * m.topk;
    const int blocks = (m.routed + DOT_BLOCK_ROWS - 1) / DOT_BLOCK_ROWS;
    L.ksplit = moe_dot_ksplit((long long)blocks * 2 * m.topk, m.hidden);
    L.wgs_per_job = (blocks + 4 / L.ksplit - 1) / (4 / L.ksplit);
    L.total_wgs = 2 * m.topk * L.wgs_per_job;
    return launch_shape<1, 4, 2, 16, 1>(L, stream);
}

int q4_dot_moe_down_launch(const MoeFuse &m, hipStream_t stream) {
    if (!moe_dot_geometry_ok(m) || dot_lds_bytes(m.routed, 1, 4, 2) > DOT_LDS_LIMIT) return -1;
    Q4DotLaunch L;
    memset(&L, 0, sizeof L);
    L.moe = m;
    L.cols = m.routed; L.tokens = 1; L.njobs = m.topk;
    const int blocks = (m.hidden + DOT_BLOCK_ROWS - 1) / DOT_BLOCK_ROWS;
    L.ksplit = moe_dot_ksplit((long long)blocks * m.topk, m.routed);
    L.wgs_per_job = (blocks + 4 / L.ksplit - 1) / (4 / L.ksplit);
    L.total_wgs = m.topk * L.wgs_per_job;
    return launch_shape<1, 4, 2, 16, 2>(L, stream);
}

}  // namespace mi355
