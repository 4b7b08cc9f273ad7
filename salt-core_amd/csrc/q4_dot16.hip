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
#include "q4_dot16_core.h"

#include <stdio.h>
#include <string.h>

namespace mi355 {
namespace {

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

// T tokens (1..4), WAVES waves of 16 rows per workgroup, MD dwords of scales per lane.  The M side of one matrix
// instruction holds two tokens; three or four tokens take a second pair of instructions per group on the same
// weight registers.
//
// PASSES: more tokens than fit beside the weight steps in LDS run as passes of T tokens inside ONE launch.
// Workgroups are numbered so that the passes over one block of rows are eight apart: the dispatcher deals
// consecutive workgroups round the device's eight partitions, so those land on one partition at about the same time
// and every pass after the first finds its weights in that partition's cache (the loads then carry the default
// cache policy instead of the non-temporal one).  The last pass may hold fewer than T tokens.
//
// WINDOWS == 2: a row too wide for the digit planes of all T tokens beside the weight steps is walked in two column
// windows (the first dot16_window_steps(steps) steps, then the rest): the workgroup builds the planes of a window,
// every wave walks the window's steps, and the planes of the next window replace them.  The weights are still read
// once, by one stream per wave that runs on across the rebuild; the accumulators carry over, so the result is what
// one window over the whole row would give.
template <int T, int WAVES, int MD, bool PASSES = false, int WINDOWS = 1>
__global__ __launch_bounds__(WAVES * 64) void q4_dot16_kernel(const Q4DotLaunch L) {
    static_assert(T >= 1 && T <= 4 && (MD == 16 || MD == 32), "tokens per pass, scale registers");
    static_assert(WINDOWS == 1 || (WINDOWS == 2 && !PASSES), "windows and passes exclude each other");
    constexpr int SETS = (T + 1) / 2;                // pairs of tokens
    constexpr int THREADS = WAVES * 64;
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    int wg = blockIdx.x, pass = 0;
    if (PASSES) {
        const int round = 8 * L.passes, within = wg % round;
        pass = within >> 3;
        wg = (wg / round) * 8 + (within & 7);
        if (wg >= L.total_wgs) return;               // the padding of the last round
    }
    const int tokens_here = PASSES ? (L.tokens_total - pass * T < T ? L.tokens_total - pass * T : T) : T;
    const Q4Job job = dot16_find_job(L, wg);
    const float *const xs = job.x + (size_t)pass * T * job.x_stride;
    float *const ys = job.y + (size_t)pass * T * job.y_stride;

    Dot16Stream<MD, PASSES ? 0 : STREAMING> stream;
    stream.setup(lane, L.cols, lds + (size_t)wave * WAVE16_LDS);
    const int window_steps = WINDOWS == 2 ? dot16_window_steps(stream.nstage) : stream.nstage;
    const int SG = window_steps * STAGE_GROUPS;      // group slots per strip in LDS (all of the row's: one window)
    uint8_t *const zero_lds = lds + WAVES * WAVE16_LDS;
    uint8_t *const img_lds = zero_lds + ZERO_BYTES;                        // [T][2 * SG][GROUP_IMAGE]
    float *const xm_lds = (float *)(img_lds + (size_t)T * 2 * SG * GROUP_IMAGE);

    const int row_base = ((wg - job.tile0) * WAVES + wave) * ROWS16;
    const bool has_rows = row_base < job.rows;       // a wave without rows still helps with the activations
    stream.bind(job.vals, job.scales, job.biases, job.rows, has_rows ? row_base : 0, 0, has_rows ? stream.nstage : 0);
    // One window: the activations are sent for first and the weights when they have arrived, so that the digit planes
    // are built while the weights are on their way (the other order, activations queued behind the first weight
    // steps, cost the batch-1 sweep 3 %).
    const ImageItems items(T, stream.ngrp);
    Q4ImageBuilder<THREADS> image;
    if (WINDOWS == 1) {
        image.request_early(tid, items, [&](int t) { return xs + (size_t)(t < tokens_here ? t : tokens_here - 1) * job.x_stride; });
        image.settle(0, items);
    }
    if (has_rows) stream.start();

    auto load_x = [&](int t, size_t column, float (&xv)[8]) {
        // a token past the last pass's end repeats the last real one (its results are not stored)
        const float *src = xs + (size_t)(t < tokens_here ? t : tokens_here - 1) * job.x_stride + column;
#pragma unroll
        for (int k = 0; k < 8; ++k) xv[k] = src[k];
    };
    if (WINDOWS == 1) {
        image.build(tid, items, SG, zero_lds, img_lds, xm_lds, load_x);
    } else {
        for (int i = tid; i < ZERO_BYTES / 4; i += THREADS) ((uint32_t *)zero_lds)[i] = 0u;
        Q4WindowBuilder<T, THREADS> front;
        front.window(stream.ngrp, stream.SG, 0, SG, SG);
        front.request(tid, load_x);
        front.build(tid, img_lds, xm_lds, load_x);
    }
    __syncthreads();
    if (WINDOWS == 1 && !has_rows) return;           // no barrier below

    const int my_token = lane >> 5;                  // of each pair
    Dot16Operand operand[SETS];
    float acc[SETS];
#pragma unroll
    for (int s = 0; s < SETS; ++s) {
        // a lane without a token (three tokens: the second pair's upper lanes) reads token 0's factors and stores nothing
        const int factor_token = 2 * s + my_token < T ? 2 * s + my_token : 0;
        const int m_tok = (lane & 15) >> 3;
        operand[s] = dot16_operand(lane, m_tok, 2 * s + m_tok < T, 2 * s + m_tok, factor_token, SG, zero_lds, img_lds, xm_lds);
        acc[s] = 0.0f;
    }
    if (WINDOWS == 1) {
        stream.run(operand, acc);
    } else {
        // every wave of the workgroup takes part in the rebuild, also one without rows.  Up to three tokens the
        // second window's activations are fetched before the walk over the first; with four, holding them across
        // the walk costs the walk more than the fetch costs the rebuild (measured: 173 against 190 us for 49
        // matrices of 2816 x 8192).
        constexpr bool AHEAD = T < 4;
        Q4WindowBuilder<T, THREADS> back;
        back.window(stream.ngrp, stream.SG, SG, (stream.nstage - window_steps) * STAGE_GROUPS, SG);
        if (AHEAD) back.request(tid, load_x);
        if (has_rows) {
            stream.settle();
            stream.walk_range(operand, acc, 0, window_steps);
        }
        __syncthreads();                             // nobody reads the first window any more
        if (!AHEAD) back.request(tid, load_x);
        back.build(tid, img_lds, xm_lds, load_x);
        __syncthreads();
        if (!has_rows) return;
        // the second window's step s lies where the first window's step s - window_steps lay
#pragma unroll
        for (int s = 0; s < SETS; ++s) {
            operand[s].digits -= (size_t)window_steps * operand[s].digits_step;
            operand[s].factors -= 2 * STAGE_GROUPS * window_steps;
        }
        stream.walk_range(operand, acc, window_steps, stream.nstage);
    }

    // the two strips of a row meet: lanes (n, 2t) and (n, 2t + 1)
#pragma unroll
    for (int s = 0; s < SETS; ++s) {
        const float other = __shfl_xor(acc[s], 16, 64);
        const int token = 2 * s + my_token;
        if (token < tokens_here && stream.my_strip == 0 && stream.n < stream.rows_here)
            ys[(size_t)token * job.y_stride + row_base + stream.n] = acc[s] + other;
    }
}

size_t dot16_lds_bytes(int cols, int tokens, int waves, int windows = 1) {
    const int steps = dot_steps(cols >> 6);
    const int sg = (windows == 2 ? dot16_window_steps(steps) : steps) * STAGE_GROUPS;
    return (size_t)waves * WAVE16_LDS + ZERO_BYTES + (size_t)tokens * 2 * sg * (GROUP_IMAGE + 8);
}

template <int T, int WAVES, int MD, bool PASSES, int WINDOWS = 1>
int launch16(const Q4DotLaunch &L, hipStream_t stream) {
    const size_t lds = dot16_lds_bytes(L.cols, T, WAVES, WINDOWS);
    static size_t raised = 0;
    if (lds > raised) {
        if (hipFuncSetAttribute((const void *)q4_dot16_kernel<T, WAVES, MD, PASSES, WINDOWS>,
                                hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess)
            return -1;
        raised = lds;
    }
    unsigned grid = (unsigned)L.total_wgs;
    if (PASSES) {
        note_kernel("q4_dot16_kernel<%d,%d,%d> x %d passes", T, WAVES, MD, L.passes);
        grid = (unsigned)((L.total_wgs + 7) / 8) * 8u * (unsigned)L.passes;
    } else if (WINDOWS == 2) {
        note_kernel("q4_dot16_kernel<%d,%d,%d> in 2 windows", T, WAVES, MD);
    } else {
        note_kernel("q4_dot16_kernel<%d,%d,%d>", T, WAVES, MD);
    }
    hipLaunchKernelGGL((q4_dot16_kernel<T, WAVES, MD, PASSES, WINDOWS>), dim3(grid), dim3(WAVES * 64), lds, stream, L);
    return hipGetLastError() == hipSuccess ? 0 : -1;
}

}  // namespace

// Waves per workgroup of the sixteen-row shape for this width and token count, or 0 when it should not be used:
// two workgroups per compute unit where the digit planes leave room, else one of twelve waves.
int q4_dot16_waves(int cols, int tokens, long long total_blocks32) {
    if (tokens > 4 || !q4_dot_takes(cols)) return 0;
    if (total_blocks32 < 2048) return 0;                                // few blocks: the 32-row kernel cuts rows instead
    if (2 * dot16_lds_bytes(cols, tokens, 8) <= DOT_LDS_LIMIT) return 8;
    if (dot16_lds_bytes(cols, tokens, 12) <= DOT_LDS_LIMIT) return 12;
    if (dot16_lds_bytes(cols, tokens, 8) <= DOT_LDS_LIMIT) return 8;    // much activation image: one workgroup of eight
    return 0;
}

// Waves per workgroup for rows walked in two column windows, or 0: the digit planes of all `tokens` tokens of half a
// row must fit beside the weight steps, and the row must have steps enough for two windows.
int q4_dot16_window_waves(int cols, int tokens, long long total_blocks32) {
    if (tokens < 3 || tokens > 4 || !q4_dot_takes(cols) || total_blocks32 < 2048) return 0;
    if (dot_steps(cols >> 6) * STAGE_GROUPS <= 32) return 0;            // only the wide-row instances exist
    if (dot16_lds_bytes(cols, tokens, 8, 2) <= DOT_LDS_LIMIT) return 8;
    return 0;
}

int q4_dot16_launch(const Q4DotLaunch &L, int waves, hipStream_t stream) {
    if (L.total_wgs < 1 || L.tokens < 1 || L.tokens > 4 || !q4_dot_takes(L.cols)) return -1;
    if (L.windows == 2) {
        if (L.passes > 1 || waves != q4_dot16_window_waves(L.cols, L.tokens, 1ll << 40)) return -1;
        if (L.tokens == 3 && waves == 8) return launch16<3, 8, 32, false, 2>(L, stream);
        if (L.tokens == 4 && waves == 8) return launch16<4, 8, 32, false, 2>(L, stream);
        return -1;
    }
    if (dot16_lds_bytes(L.cols, L.tokens, waves) > DOT_LDS_LIMIT) return -1;
    const int md = dot_steps(L.cols >> 6) * STAGE_GROUPS <= 32 ? 16 : 32;
    if (L.passes > 1) {
        if (L.tokens_total <= (L.passes - 1) * L.tokens || L.tokens_total > L.passes * L.tokens) return -1;
#define DOT16_PASSES(TT, WW) \
        if (L.tokens == TT && waves == WW) \
            return md == 16 ? launch16<TT, WW, 16, true>(L, stream) : launch16<TT, WW, 32, true>(L, stream)
        DOT16_PASSES(4, 8); DOT16_PASSES(4, 12);
#undef DOT16_PASSES
        return -1;
    }
#define DOT16_CASE(TT, WW) \
    if (L.tokens == TT && waves == WW) \
        return md == 16 ? launch16<TT, WW, 16, false>(L, stream) : launch16<TT, WW, 32, false>(L, stream)
    DOT16_CASE(1, 8); DOT16_CASE(2, 8); DOT16_CASE(3, 8); DOT16_CASE(4, 8);
    DOT16_CASE(1, 12); DOT16_CASE(2, 12); DOT16_CASE(3, 12); DOT16_CASE(4, 12);
#undef DOT16_CASE
    return -1;
}

// Whether q4_dot16_launch serves `passes` passes of `tokens` tokens with `waves` waves per workgroup.
bool q4_dot16_takes_passes(int tokens, int waves) {
    return tokens == 4 && (waves == 8 || waves == 12);
}

}  // namespace mi355
