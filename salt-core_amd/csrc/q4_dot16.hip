// Affine-Q4 decode matvec, tolerance class, for launches with many blocks (one to four tokens): the arithmetic and
// the bound of q4_dot.hip on blocks of sixteen rows.
//
// Why a second shape: a step of q4_dot.hip (32 rows, 8 KiB) keeps a wave busy for about as long as two steps take to
// arrive, and LDS holds only eight such waves per compute unit, so the arithmetic's latencies (LDS reads, dependent
// matrix instructions) are exposed.  Here a wave owns 16 rows and a step is 4 KiB: sixteen waves fit, the matrix
// instruction is v_mfma_i32_16x16x64_i8 (half the matrix time per weight, four accumulator registers instead of
// sixteen), and the same 128 KiB of steps are in flight per compute unit.
//
// Matrix instruction as dot-product bank: N = 16 weight rows; K = 64 = sixteen columns of each half of one group
// of each of the two strips (lane l = (row l % 16, k-slice l / 16): strip (l / 32), half (l / 16) % 2); M = 16 rows
// of digits, row m = (token m / 8, strip (m / 4) % 2, plane m % 4), zero outside its own strip's k-slices.  Two
// instructions cover a group of each strip; the plane sums of lane (row, strip [+ 2 * token]) follow as in
// q4_dot.hip.
#include "dot_common.h"
#include "q4_image.h"

#include <stdio.h>
#include <string.h>

namespace mi355 {
namespace {

constexpr int ROWS16 = 16;                   // rows per block = N of the matrix instruction
constexpr int STEP16_BYTES = 4096;           // 2 strips x 16 rows x 128 bytes
constexpr int LOADS16 = 4;                   // weight loads per step

__device__ __forceinline__ Q4Job dot16_find_job(const Q4DotLaunch &L, int wg) {
    if (L.table == nullptr && L.njobs <= 1) return L.one;
    const uniform_u64_ptr words =
        L.table ? (uniform_u64_ptr)(uintptr_t)L.table
                : (uniform_u64_ptr)((const char __attribute__((address_space(4))) *)__builtin_amdgcn_kernarg_segment_ptr() +
                                    offsetof(Q4DotLaunch, inline_jobs));
    int lo = 0, hi = L.njobs - 1;
    if (L.wgs_per_job > 0) {
        lo = wg / L.wgs_per_job;
    } else {
        while (lo < hi) {
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

// T tokens (1..4), WAVES waves of 16 rows per workgroup, MD dwords of scales per lane.  Two steps of LDS per wave.
// The M side of one matrix instruction holds two tokens; three or four tokens take a second pair of instructions per
// group on the same weight registers.
template <int T, int WAVES, int MD>
__global__ __launch_bounds__(WAVES * 64) void q4_dot16_kernel(const Q4DotLaunch L) {
    static_assert(T >= 1 && T <= 4 && (MD == 16 || MD == 32), "tokens per pass, scale registers");
    constexpr int SETS = (T + 1) / 2;                // pairs of tokens
    constexpr int STAGES = 2;
    constexpr int WAVE_LDS = STAGES * STEP16_BYTES;
    constexpr int THREADS = WAVES * 64;
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const Q4Job job = dot16_find_job(L, blockIdx.x);

    const int C = L.cols;
    const int ngrp = C >> 6;
    const int nstage = dot_steps(ngrp);
    const int SG = nstage * STAGE_GROUPS;            // groups of strip 0; strip 1 holds the remaining ngrp - SG
    const uint32_t row_bytes = (uint32_t)C >> 1;
    const int whole_steps = (ngrp - SG) / STAGE_GROUPS;
    // a lane's window of scales: meta_groups groups of its row from its strip's first group, moved left at the row's end
    const int meta_groups = 2 * MD < (ngrp & ~7) ? 2 * MD : ngrp & ~7;
    const int window1 = SG <= ngrp - meta_groups ? SG : ngrp - meta_groups;
    const int shift1 = SG - window1;                 // strip 0's window starts at group 0

    uint8_t *const w_lds = lds;                                            // [WAVES][STAGES][STEP16_BYTES]
    uint8_t *const zero_lds = lds + WAVES * WAVE_LDS;
    uint8_t *const img_lds = zero_lds + ZERO_BYTES;                        // [T][2 * SG][GROUP_IMAGE]
    float *const xm_lds = (float *)(img_lds + (size_t)T * 2 * SG * GROUP_IMAGE);

    const int row_base = (((int)blockIdx.x - job.tile0) * WAVES + wave) * ROWS16;
    const bool has_rows = row_base < job.rows;
    const int rows_here = !has_rows ? 1 : (job.rows - row_base < ROWS16 ? job.rows - row_base : ROWS16);
    const int total_steps = has_rows ? nstage : 0;

    // ---------------------------------------------------------------- per-lane geometry
    // loads: load k of a step covers strip k / 2, rows 8 (k % 2) .. + 7; lane i lands in slot 64 k + i, that is piece
    // (strip * 16 + row), position i % 8, which receives segment (i % 8) ^ swizzle(piece)
    uint8_t *const my_lds = w_lds + (size_t)wave * WAVE_LDS;
    int src_rowi[LOADS16];
    uint32_t src_col[LOADS16], src_off[LOADS16];
#pragma unroll
    for (int k = 0; k < LOADS16; ++k) {
        const int strip = k >> 1;
        const int row = (k & 1) * 8 + (lane >> 3);
        const int piece = strip * 16 + row;
        const int seg = (lane & 7) ^ swizzle(piece);
        src_rowi[k] = row;
        src_col[k] = (uint32_t)(strip * SG) * 32u + (uint32_t)seg * 16u;
        src_off[k] = (uint32_t)row * row_bytes + src_col[k];
    }
    // reads: lane (n, kq) takes half (kq % 2) of every group of strip kq / 2 of row n
    const int n = lane & 15, kq = lane >> 4;
    const int my_piece = (kq >> 1) * 16 + n;
    uint32_t rd_off[STAGE_GROUPS];
#pragma unroll
    for (int u = 0; u < STAGE_GROUPS; ++u)
        rd_off[u] = (uint32_t)my_piece * 128u + (uint32_t)((2 * u + (kq & 1)) ^ swizzle(my_piece)) * 16u;
    // results: lane (n, mq) holds row n's plane sums of strip mq % 2, token mq / 2 of each pair of tokens
    const int mq = kq;
    const int my_strip = mq & 1, my_token = mq >> 1;
    const bool no_bias = job.biases == nullptr;
    // digit planes: row m = l % 16 of the M side is (token m / 8, strip (m / 4) % 2, plane m % 4); it carries digits in
    // the two k-slices of its own strip
    const int m_tok = n >> 3, m_strip = (n >> 2) & 1, m_plane = n & 3;
    const uint8_t *a_base[SETS];
    uint32_t a_step[SETS];
    const float *xm_ptr[SETS];
#pragma unroll
    for (int s = 0; s < SETS; ++s) {
        const bool has_digits = 2 * s + m_tok < T && m_strip == (kq >> 1);
        a_base[s] = has_digits
            ? img_lds + ((size_t)((2 * s + m_tok) * 2 * SG + m_strip * SG) * 16 + 2 * (kq & 1) * 4 + m_plane) * 16
            : zero_lds + 64;
        a_step[s] = has_digits ? STAGE_GROUPS * GROUP_IMAGE : 0u;
        // a lane without a token (three tokens: the second pair's upper lanes) reads token 0's factors and stores nothing
        const int tok = 2 * s + my_token < T ? 2 * s + my_token : 0;
        xm_ptr[s] = xm_lds + 2 * (tok * 2 * SG + my_strip * SG);
    }

    // ---------------------------------------------------------------- loads
    typedef uint32_t MetaVec __attribute__((ext_vector_type(MD)));
    MetaRegs<MD> scales_r, biases_r;
    MetaVec scales_v, biases_v;
    auto issue_meta = [&]() {
        const int row = n < rows_here ? n : rows_here - 1;
        const size_t at = ((size_t)(row_base + row) * ngrp + (my_strip ? window1 : 0)) * 2;
#pragma unroll
        for (int q = 0; q < MD / 4; ++q) {
            const int piece = 8 * q < meta_groups ? q : (meta_groups - 1) / 8;
            scales_r.q[q] = load_meta16(job.scales + at + 16 * piece);
            biases_r.q[q] = load_meta16((no_bias ? job.scales : job.biases) + at + 16 * piece);
        }
    };
    const uint8_t *const block_vals = job.vals + (size_t)row_base * row_bytes;
    auto issue_step = [&](int st, int slot) {
        uint8_t *const stage = my_lds + slot * STEP16_BYTES;
        const uint32_t advance = (uint32_t)st * (STAGE_GROUPS * 32);
        if (rows_here == ROWS16 && st < whole_steps) {
#pragma unroll
            for (int k = 0; k < LOADS16; ++k)
                __builtin_amdgcn_global_load_lds((global_u128_ptr)(uintptr_t)(block_vals + advance + src_off[k]),
                                                 (lds_void_ptr)(stage + k * 1024), 16, 0, STREAMING);
        } else {
#pragma unroll
            for (int k = 0; k < LOADS16; ++k) {
                const int row = src_rowi[k] < rows_here ? src_rowi[k] : rows_here - 1;
                uint32_t col = src_col[k] + advance;
                col = col <= row_bytes - 16 ? col : row_bytes - 16;
                __builtin_amdgcn_global_load_lds((global_u128_ptr)(uintptr_t)(block_vals + ((uint32_t)row * row_bytes + col)),
                                                 (lds_void_ptr)(stage + k * 1024), 16, 0, STREAMING);
            }
        }
    };

    // ---------------------------------------------------------------- arithmetic of one step
    float acc[SETS];
#pragma unroll
    for (int s = 0; s < SETS; ++s) acc[s] = 0.0f;
    struct StepWeights { u32x4 group[STAGE_GROUPS]; };
    auto fetch = [&](int slot, StepWeights &w) {
        const uint8_t *stage = my_lds + slot * STEP16_BYTES;
#pragma unroll
        for (int u = 0; u < STAGE_GROUPS; ++u) w.group[u] = *(const u32x4 *)(stage + rd_off[u]);
    };
    auto consume = [&](int st, const StepWeights &w) {
        // the step's four scales and four biases of the lane's result strip (register indexing, wave-uniform index
        // per strip)
        float scale[STAGE_GROUPS], bias[STAGE_GROUPS];
        {
            const int last = MD - 2;
            const int at0 = 2 * st, at1 = 2 * st + (shift1 >> 1);
            const int i0 = at0 < last ? at0 : last, i1 = at1 < last ? at1 : last;
            uint32_t s_lo = scales_v[i0], s_hi = scales_v[i0 + 1], b_lo = biases_v[i0], b_hi = biases_v[i0 + 1];
            if (i1 != i0) {
                const uint32_t s_lo1 = scales_v[i1], s_hi1 = scales_v[i1 + 1], b_lo1 = biases_v[i1], b_hi1 = biases_v[i1 + 1];
                s_lo = my_strip ? s_lo1 : s_lo; s_hi = my_strip ? s_hi1 : s_hi;
                b_lo = my_strip ? b_lo1 : b_lo; b_hi = my_strip ? b_hi1 : b_hi;
            }
            scale[0] = __uint_as_float(s_lo << 16); scale[1] = __uint_as_float(s_lo & 0xffff0000u);
            scale[2] = __uint_as_float(s_hi << 16); scale[3] = __uint_as_float(s_hi & 0xffff0000u);
            bias[0] = __uint_as_float(b_lo << 16); bias[1] = __uint_as_float(b_lo & 0xffff0000u);
            bias[2] = __uint_as_float(b_hi << 16); bias[3] = __uint_as_float(b_hi & 0xffff0000u);
            if (no_bias) { bias[0] = bias[1] = bias[2] = bias[3] = 0.0f; }
        }
        // unpacked codes of the step: the operands of both instructions of every group, shared by the token pairs
        v4i b[STAGE_GROUPS][2];
#pragma unroll
        for (int u = 0; u < STAGE_GROUPS; ++u)
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                const uint32_t lo = j ? w.group[u].z : w.group[u].x, hi = j ? w.group[u].w : w.group[u].y;
                b[u][j].x = (int)(lo & 0x0f0f0f0fu);
                b[u][j].y = (int)((lo >> 4) & 0x0f0f0f0fu);
                b[u][j].z = (int)(hi & 0x0f0f0f0fu);
                b[u][j].w = (int)((hi >> 4) & 0x0f0f0f0fu);
            }
#pragma unroll
        for (int s = 0; s < SETS; ++s) {
            const uint8_t *a_ptr = a_base[s] + (uint32_t)st * a_step[s];
            const f32x4 xm_a = *(const f32x4 *)(xm_ptr[s] + 2 * (st * STAGE_GROUPS));
            const f32x4 xm_b = *(const f32x4 *)(xm_ptr[s] + 2 * (st * STAGE_GROUPS) + 4);
            const float xm[8] = {xm_a.x, xm_a.y, xm_a.z, xm_a.w, xm_b.x, xm_b.y, xm_b.z, xm_b.w};
            v4i d[STAGE_GROUPS];
#pragma unroll
            for (int u = 0; u < STAGE_GROUPS; ++u) d[u] = v4i{0, 0, 0, 0};
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                v4i a[STAGE_GROUPS];
#pragma unroll
                for (int u = 0; u < STAGE_GROUPS; ++u) a[u] = *(const v4i *)(a_ptr + u * GROUP_IMAGE + j * 64);
#pragma unroll
                for (int u = 0; u < STAGE_GROUPS; ++u) d[u] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a[u], b[u][j], d[u], 0, 0, 0);
            }
#pragma unroll
            for (int u = 0; u < STAGE_GROUPS; ++u) {
                const int lo = d[u].x + (d[u].y << 8);
                const int hi = d[u].z + (d[u].w << 8);
                const float f = __builtin_fmaf((float)hi, 65536.0f, (float)lo);
                acc[s] = __builtin_fmaf(scale[u] * xm[2 * u], f, acc[s]);
                acc[s] = __builtin_fmaf(bias[u], xm[2 * u + 1], acc[s]);
            }
        }
    };

    // ---------------------------------------------------------------- main sequence (as in q4_dot.hip)
    if (has_rows) {
        issue_meta();
#pragma unroll
        for (int g = 0; g < STAGES; ++g)
            if (g < total_steps) issue_step(g, g);
    }
    build_q4_image<T, THREADS>(tid, ngrp, SG, zero_lds, img_lds, xm_lds, [&](int t, size_t column, float (&xv)[4]) {
        const float *src = job.x + (size_t)t * job.x_stride + column;
#pragma unroll
        for (int k = 0; k < 4; ++k) xv[k] = src[k];
    });
    __syncthreads();
    if (!has_rows) return;                           // no barrier below
#pragma unroll
    for (int q = 0; q < MD / 4; ++q) {
        wait_meta(scales_r.q[q]);
        wait_meta(biases_r.q[q]);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            scales_v[4 * q + e] = scales_r.q[q][e];
            biases_v[4 * q + e] = biases_r.q[q][e];
        }
    }
    if (shift1 & 1) {
        // strip 1's window starts an odd number of groups before the strip: move its lanes' values down by one group
#pragma unroll
        for (int i = 0; i < MD; ++i) {
            const uint32_t s_next = i + 1 < MD ? scales_v[i + 1] : 0u, b_next = i + 1 < MD ? biases_v[i + 1] : 0u;
            const uint32_t s_moved = __builtin_amdgcn_alignbit(s_next, scales_v[i], 16);
            const uint32_t b_moved = __builtin_amdgcn_alignbit(b_next, biases_v[i], 16);
            scales_v[i] = my_strip ? s_moved : scales_v[i];
            biases_v[i] = my_strip ? b_moved : biases_v[i];
        }
    }
    for (int base = 0; base < total_steps; base += STAGES) {
        const bool more = static_steps(std::make_integer_sequence<int, STAGES>{}, [&](auto step_in_turn) {
            constexpr int r = decltype(step_in_turn)::value;
            const int g = base + r;
            if (g >= total_steps) return false;
            if (g + 1 < total_steps) wait_vm<LOADS16>(); else wait_vm<0>();
            StepWeights w;
            fetch(r, w);
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");          // the reads have returned before the slot is refilled
            if (g + STAGES < total_steps) issue_step(g + STAGES, r);
            consume(g, w);
            return true;
        });
        if (!more) break;
    }
    // the two strips of a row meet: lanes (n, 2t) and (n, 2t + 1)
#pragma unroll
    for (int s = 0; s < SETS; ++s) {
        const float other = __shfl_xor(acc[s], 16, 64);
        const int token = 2 * s + my_token;
        if (token < T && my_strip == 0 && n < rows_here) job.y[(size_t)token * job.y_stride + row_base + n] = acc[s] + other;
    }
}

size_t dot16_lds_bytes(int cols, int tokens, int waves) {
    const int sg = dot_steps(cols >> 6) * STAGE_GROUPS;
    return (size_t)waves * 2 * STEP16_BYTES + ZERO_BYTES + (size_t)tokens * 2 * sg * (GROUP_IMAGE + 8);
}

template <int T, int WAVES, int MD>
int launch16(const Q4DotLaunch &L, hipStream_t stream) {
    const size_t lds = dot16_lds_bytes(L.cols, T, WAVES);
    static size_t raised = 0;
    if (lds > raised) {
        if (hipFuncSetAttribute((const void *)q4_dot16_kernel<T, WAVES, MD>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                (int)lds) != hipSuccess)
            return -1;
        raised = lds;
    }
    note_kernel("q4_dot16_kernel<%d,%d,%d>", T, WAVES, MD);
    hipLaunchKernelGGL((q4_dot16_kernel<T, WAVES, MD>), dim3(L.total_wgs), dim3(WAVES * 64), lds, stream, L);
    return hipGetLastError() == hipSuccess ? 0 : -1;
}

}  // namespace

// Waves per workgroup of the sixteen-row shape for this width and token count, or 0 when it should not be used:
// two workgroups per compute unit where the digit planes leave room, else one of twelve waves.
int q4_dot16_waves(int cols, int tokens, long long total_blocks32) {
    static const int want = env_int("SALT_MI355_DOT16", -1);           // 0 forbids the shape, 8 / 12 force it
    if (want == 0 || tokens > 4 || !q4_dot_takes(cols)) return 0;
    if (want != 8 && want != 12 && total_blocks32 < 2048) return 0;     // few blocks: the 32-row kernel cuts rows instead
    if ((want == -1 || want == 8) && 2 * dot16_lds_bytes(cols, tokens, 8) <= DOT_LDS_LIMIT) return 8;
    if ((want == -1 || want == 12) && dot16_lds_bytes(cols, tokens, 12) <= DOT_LDS_LIMIT) return 12;
    return 0;
}

int q4_dot16_launch(const Q4DotLaunch &L, int waves, hipStream_t stream) {
    if (L.total_wgs < 1 || L.tokens < 1 || L.tokens > 4 || !q4_dot_takes(L.cols)) return -1;
    if (dot16_lds_bytes(L.cols, L.tokens, waves) > DOT_LDS_LIMIT) return -1;
    const int md = dot_steps(L.cols >> 6) * STAGE_GROUPS <= 32 ? 16 : 32;
#define DOT16_CASE(TT, WW) \
    if (L.tokens == TT && waves == WW) return md == 16 ? launch16<TT, WW, 16>(L, stream) : launch16<TT, WW, 32>(L, stream)
    DOT16_CASE(1, 8); DOT16_CASE(2, 8); DOT16_CASE(3, 8); DOT16_CASE(4, 8);
    DOT16_CASE(1, 12); DOT16_CASE(2, 12); DOT16_CASE(3, 12); DOT16_CASE(4, 12);
#undef DOT16_CASE
    return -1;
}

}  // namespace mi355
