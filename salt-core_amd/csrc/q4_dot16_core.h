// One wave's stream of the sixteen-row tolerance-class affine-Q4 kernels (q4_dot16.hip, moe_dot16.hip): the wave
// owns 16 rows of one matrix, walks the steps [step_lo, step_hi) of their two strips (4 KiB per step, straight into
// LDS, two steps in flight), multiplies with digit planes that the caller has placed in LDS (q4_image.h) and returns
// per lane the sum of its result strip.
//
// Lane roles.  As reader of weights, lane l = (row l % 16, k-slice l / 16): strip (l / 32), half (l / 16) % 2 of every
// group.  As holder of results, lane l = (row l % 16, mq = l / 16): strip mq % 2, token mq / 2 of each pair of tokens.
// The M side of v_mfma_i32_16x16x64_i8 holds row m = (token m / 8, strip (m / 4) % 2, plane m % 4) of digits, zero
// outside its own strip's k-slices.
#pragma once

#include "dot_common.h"
#include "q4_image.h"

namespace mi355 {
namespace {

constexpr int ROWS16 = 16;                   // rows per block = N of the matrix instruction
constexpr int STEP16_BYTES = 4096;           // 2 strips x 16 rows x 128 bytes
constexpr int LOADS16 = 4;                   // weight loads per step
constexpr int WAVE16_LDS = 2 * STEP16_BYTES; // two steps per wave

// Steps of the first of two column windows of a row of `steps` steps: at least half of them, and even (a window
// starts on the first of the two step slots).
__host__ __device__ constexpr int dot16_window_steps(int steps) { return ((steps + 1) / 2 + 1) & ~1; }

// Where a lane finds the digits and the per-group factors of one pair of tokens.
struct Dot16Operand {
    const uint8_t *digits;    // the lane's 16-byte piece of step 0, group 0, first quarter (or the zero region)
    uint32_t digits_step;     // bytes from one step to the next (0 for the zero region)
    const float *factors;     // (power of two, sum) of the lane's result strip and token, group 0
};

// Address of the digits that lane (m = lane % 16, k-slice lane / 16) feeds to the matrix instruction for `token`, or
// the zero region when the lane's M row carries none (another strip's row, or no such token).
__device__ __forceinline__ Dot16Operand dot16_operand(int lane, int token_of_pair, bool token_exists, int image_token,
                                                      int factor_token, int SG, const uint8_t *zero_lds,
                                                      const uint8_t *img_lds, const float *xm_lds) {
    const int n = lane & 15, kq = lane >> 4;
    const int m_tok = n >> 3, m_strip = (n >> 2) & 1, m_plane = n & 3;
    const bool has_digits = token_exists && m_tok == token_of_pair && m_strip == (kq >> 1);
    Dot16Operand op;
    op.digits = has_digits
        ? img_lds + ((size_t)(image_token * 2 * SG + m_strip * SG) * 16 + 2 * (kq & 1) * 4 + m_plane) * 16
        : zero_lds + 64;              // a bank group that no digit plane of the same read occupies
    op.digits_step = has_digits ? STAGE_GROUPS * GROUP_IMAGE : 0u;
    op.factors = xm_lds + 2 * (factor_token * 2 * SG + (kq & 1) * SG);
    return op;
}

// POLICY: cache policy of the weight loads (STREAMING = non-temporal: every byte is read once by this launch).
template <int MD, int POLICY = STREAMING>
struct Dot16Stream {
    // what the wave walks
    const uint8_t *vals, *scales, *biases;       // biases may be null
    int row_base, rows_here;                     // its rows of the matrix (1..16 of them)
    int ngrp, nstage, SG, whole_steps;
    int step_lo, step_hi;
    uint32_t row_bytes;
    uint8_t *my_lds;                             // WAVE16_LDS bytes: the two slots steps alternate between ...
    uint8_t *slot_lds[2];                        // ... unless the caller places them elsewhere (place_slots)
    // per-lane geometry
    int lane, n, kq, my_strip;
    int src_rowi[LOADS16];
    uint32_t src_col[LOADS16], src_off[LOADS16], rd_off[STAGE_GROUPS];
    int meta_groups, window0, window1, shift0, shift1;
    MetaRegs<MD> scales_r, biases_r;
    typedef uint32_t MetaVec __attribute__((ext_vector_type(MD)));
    MetaVec scales_v, biases_v;                  // the same values as one indexable vector, valid after settle()

    __device__ __forceinline__ void setup(int lane_, int cols, uint8_t *lds_of_wave) {
        lane = lane_;
        n = lane & 15; kq = lane >> 4; my_strip = kq & 1;
        my_lds = lds_of_wave;
        slot_lds[0] = lds_of_wave; slot_lds[1] = lds_of_wave + STEP16_BYTES;
        ngrp = cols >> 6;
        nstage = dot_steps(ngrp);
        SG = nstage * STAGE_GROUPS;              // groups of strip 0; strip 1 holds the remaining ngrp - SG
        row_bytes = (uint32_t)cols >> 1;
        whole_steps = (ngrp - SG) / STAGE_GROUPS;
        // loads: load k of a step covers strip k / 2, rows 8 (k % 2) .. + 7; lane i lands in slot 64 k + i, that is
        // piece (strip * 16 + row), position i % 8, which receives segment (i % 8) ^ swizzle(piece)
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
        const int my_piece = (kq >> 1) * 16 + n;
#pragma unroll
        for (int u = 0; u < STAGE_GROUPS; ++u)
            rd_off[u] = (uint32_t)my_piece * 128u + (uint32_t)((2 * u + (kq & 1)) ^ swizzle(my_piece)) * 16u;
    }

    // The matrix, the wave's rows and its steps.  A lane keeps the scales of meta_groups groups of its row in
    // registers: a window from its result strip's first group of the wave's steps, moved left at the row's end.
    __device__ __forceinline__ void bind(const uint8_t *vals_, const uint8_t *scales_, const uint8_t *biases_, int rows,
                                         int first_row, int first_step, int end_step) {
        vals = vals_; scales = scales_; biases = biases_;
        row_base = first_row;
        rows_here = rows - first_row < ROWS16 ? rows - first_row : ROWS16;
        if (rows_here < 1) rows_here = 1;
        step_lo = first_step; step_hi = end_step;
        meta_groups = 2 * MD < (ngrp & ~7) ? 2 * MD : ngrp & ~7;
        const int want0 = step_lo * STAGE_GROUPS, want1 = SG + step_lo * STAGE_GROUPS;
        window0 = want0 <= ngrp - meta_groups ? want0 : ngrp - meta_groups;
        window1 = want1 <= ngrp - meta_groups ? want1 : ngrp - meta_groups;
        shift0 = want0 - window0; shift1 = want1 - window1;
    }

    __device__ __forceinline__ void issue_step(int st, int slot) {
        uint8_t *const stage = slot_lds[slot];
        const uint8_t *const block_vals = vals + (size_t)row_base * row_bytes;
        const uint32_t advance = (uint32_t)st * (STAGE_GROUPS * 32);
        if (rows_here == ROWS16 && st < whole_steps) {
            // a wave-uniform base that advances with the step plus a fixed 32-bit offset per lane
#pragma unroll
            for (int k = 0; k < LOADS16; ++k)
                __builtin_amdgcn_global_load_lds((global_u128_ptr)(uintptr_t)(block_vals + advance + src_off[k]),
                                                 (lds_void_ptr)(stage + k * 1024), 16, 0, POLICY);
        } else {
            // the matrix ends inside this block, or strip 1 ends inside this step or before it: stay inside
#pragma unroll
            for (int k = 0; k < LOADS16; ++k) {
                const int row = src_rowi[k] < rows_here ? src_rowi[k] : rows_here - 1;
                uint32_t col = src_col[k] + advance;
                col = col <= row_bytes - 16 ? col : row_bytes - 16;
                __builtin_amdgcn_global_load_lds((global_u128_ptr)(uintptr_t)(block_vals + ((uint32_t)row * row_bytes + col)),
                                                 (lds_void_ptr)(stage + k * 1024), 16, 0, POLICY);
            }
        }
    }

    __device__ __forceinline__ void place_slots(uint8_t *even_steps, uint8_t *odd_steps) {
        slot_lds[0] = even_steps; slot_lds[1] = odd_steps;
    }

    // The scales and biases of the wave's rows go out.
    __device__ __forceinline__ void issue_meta() {
        const int row = n < rows_here ? n : rows_here - 1;
        const size_t at = ((size_t)(row_base + row) * ngrp + (my_strip ? window1 : window0)) * 2;
        const uint8_t *bias_src = biases ? biases : scales;           // the load happens either way; its result is dropped
#pragma unroll
        for (int q = 0; q < MD / 4; ++q) {
            const int piece = 8 * q < meta_groups ? q : (meta_groups - 1) / 8;
            scales_r.q[q] = load_meta16(scales + at + 16 * piece);
            biases_r.q[q] = load_meta16(bias_src + at + 16 * piece);
        }
    }

    // Scales, biases and the first two steps go out: none of them depends on the activations, so the caller builds
    // the digit planes while they are on their way.
    __device__ __forceinline__ void start() {
        issue_meta();
#pragma unroll
        for (int g = 0; g < 2; ++g)
            if (step_lo + g < step_hi) issue_step(step_lo + g, g);
    }

    // The stream itself, after the digit planes are in place (a barrier lies between start() and run()).  acc[s] of
    // lane (n, mq) receives row n's sum over the wave's steps of strip mq % 2 for token mq / 2 of pair s.
    template <int SETS>
    __device__ __forceinline__ void run(const Dot16Operand (&operand)[SETS], float (&acc)[SETS]) {
        settle();
        walk(operand, acc);
    }

    // Waits for the scales and biases, the only loads that return to registers, together with everything else the
    // wave has in flight.
    __device__ __forceinline__ void settle() {
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
        if ((shift0 | shift1) & 1) {
            // a window that starts an odd number of groups before the first step: move the lane's values down by one
            // group (16 bits), so that a step's four again fill two whole registers
            const bool odd = ((my_strip ? shift1 : shift0) & 1) != 0;
#pragma unroll
            for (int i = 0; i < MD; ++i) {
                const uint32_t s_next = i + 1 < MD ? scales_v[i + 1] : 0u, b_next = i + 1 < MD ? biases_v[i + 1] : 0u;
                const uint32_t s_moved = __builtin_amdgcn_alignbit(s_next, scales_v[i], 16);
                const uint32_t b_moved = __builtin_amdgcn_alignbit(b_next, biases_v[i], 16);
                scales_v[i] = odd ? s_moved : scales_v[i];
                biases_v[i] = odd ? b_moved : biases_v[i];
            }
        }
    }

    // The walk over the wave's steps, after settle(); the first two steps have been issued.
    template <int SETS>
    __device__ __forceinline__ void walk(const Dot16Operand (&operand)[SETS], float (&acc)[SETS]) {
        walk_range(operand, acc, 0, step_hi - step_lo);
    }

    // Steps [from, to) of the wave's steps, counted from step_lo; `from` is even.  Steps from and from + 1 have been
    // issued (by start() or by the range before); the range issues up to two steps past its own end when the wave
    // has them, so that ranges follow each other without a gap in the stream.
    template <int SETS>
    __device__ __forceinline__ void walk_range(const Dot16Operand (&operand)[SETS], float (&acc)[SETS], int from, int to) {
        const bool no_bias = biases == nullptr;
        const int total_steps = step_hi - step_lo;
        struct StepWeights { u32x4 group[STAGE_GROUPS]; };

        auto consume = [&](int st, const StepWeights &w) {
            // the step's four scales and four biases of the lane's result strip: register indexing at a wave-uniform
            // index per strip (groups past the row's end meet zero digits; they take whatever the clamped index yields)
            float scale[STAGE_GROUPS], bias[STAGE_GROUPS];
            {
                // A step's four groups are two dwords; past the registers' end (a step that straddles the row's end:
                // its real groups are in the last dword, the rest meet zero digits) each index is held back on its own
                const int at0 = 2 * (st - step_lo) + (shift0 >> 1), at1 = 2 * (st - step_lo) + (shift1 >> 1);
                const int lo0 = at0 < MD - 1 ? at0 : MD - 1, hi0 = at0 + 1 < MD - 1 ? at0 + 1 : MD - 1;
                const int lo1 = at1 < MD - 1 ? at1 : MD - 1, hi1 = at1 + 1 < MD - 1 ? at1 + 1 : MD - 1;
                uint32_t s_lo = scales_v[lo0], s_hi = scales_v[hi0], b_lo = biases_v[lo0], b_hi = biases_v[hi0];
                if (at1 != at0) {                  // uniform
                    const uint32_t s_lo1 = scales_v[lo1], s_hi1 = scales_v[hi1], b_lo1 = biases_v[lo1], b_hi1 = biases_v[hi1];
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
                const uint8_t *a_ptr = operand[s].digits + (uint32_t)st * operand[s].digits_step;
                // read as native vectors: an LDS read without type information is made to wait for every outstanding
                // direct-to-LDS load by the compiler
                const f32x4 xm_a = *(const f32x4 *)(operand[s].factors + 2 * (st * STAGE_GROUPS));
                const f32x4 xm_b = *(const f32x4 *)(operand[s].factors + 2 * (st * STAGE_GROUPS) + 4);
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
                    for (int u = 0; u < STAGE_GROUPS; ++u)
                        d[u] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a[u], b[u][j], d[u], 0, 0, 0);
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

        // Loads go out in step order, four per step, two steps ahead: a step's slot is refilled as soon as its
        // weights sit in registers.  Direct-to-LDS loads complete in issue order, so when step g is waited for, what
        // may still be in flight is the step behind it.
        for (int base = from; base < to; base += 2) {
            const bool more = static_steps(std::make_integer_sequence<int, 2>{}, [&](auto step_in_turn) {
                constexpr int r = decltype(step_in_turn)::value;
                const int g = base + r;
                if (g >= to) return false;
                if (g + 1 < total_steps) wait_vm<LOADS16>(); else wait_vm<0>();
                StepWeights w;
                const uint8_t *stage = slot_lds[r];
#pragma unroll
                for (int u = 0; u < STAGE_GROUPS; ++u) w.group[u] = *(const u32x4 *)(stage + rd_off[u]);
                asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");      // the reads have returned before the slot is refilled
                if (g + 2 < total_steps) issue_step(step_lo + g + 2, r);
                consume(step_lo + g, w);
                return true;
            });
            if (!more) break;
        }
    }
};

}  // namespace
}  // namespace mi355
