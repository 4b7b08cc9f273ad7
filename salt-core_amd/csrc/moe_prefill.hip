// Grouped prefill MoE on the device (tolerance class for the values, exact
// for the bucketing).
//
// reference src/moe_group.c:24-97 (validation: expert ids in range, finite
// weights, no expert twice in a token), :138-184 (rows of a wave of experts:
// ascending expert, then token, then rank; outputs scattered back to
// [token][rank] slots), :211-224 (out[token] = sum over rank of slot * weight,
// from +0, rank ascending).  The per-expert arithmetic (gate, up, gelu*up,
// down: gemma4_text.c:8749-9137) runs on the MFMA matmul of q4_mfma.hip, so
// values carry that kernel's tolerance; which row goes where is integer work
// and identical to the reference.
#include "device_math.h"
#include "mi355_internal.h"

#include <string.h>

namespace mi355 {
namespace {

constexpr int MAX_EXPERTS = 1024;

struct PrefillPlan {            // device ints produced by the count and scan kernels
    int status;                 // 0 ok, -1 the selection is invalid
    int gate_up_jobs, down_jobs;
    int gate_up_tiles, down_tiles;
};

// Exclusive prefix sum over the threads of a workgroup (blockDim a multiple of 64, at most 1024).
__device__ __forceinline__ int block_exclusive_scan(int v, int *wave_totals, int *total) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, waves = blockDim.x >> 6;
    int incl = v;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
        const int up = __shfl_up(incl, off, 64);
        if (lane >= off) incl += up;
    }
    __syncthreads();                                   // wave_totals may still be read from an earlier call
    if (lane == 63) wave_totals[wave] = incl;
    __syncthreads();
    int before = 0, all = 0;
    for (int w = 0; w < waves; ++w) {
        const int t = wave_totals[w];
        before += w < wave ? t : 0;
        all += t;
    }
    if (total) *total = all;
    return before + incl - v;
}

// one thread per token: validate, count per expert in LDS, then one global add per expert and workgroup
__global__ __launch_bounds__(256) void group_count_kernel(const int *__restrict__ selected,
                                                          const float *__restrict__ weights, int tokens, int topk,
                                                          int n_experts, int *__restrict__ counts,
                                                          PrefillPlan *__restrict__ plan) {
    __shared__ int s_count[MAX_EXPERTS];
    for (int e = threadIdx.x; e < n_experts; e += blockDim.x) s_count[e] = 0;
    __syncthreads();
    const int t = blockIdx.x * blockDim.x + threadIdx.x;
    if (t < tokens) {
        bool ok = true;
        for (int k = 0; k < topk; ++k) {
            const int e = selected[(size_t)t * topk + k];
            const float w = weights[(size_t)t * topk + k];
            if (e < 0 || e >= n_experts || !(__builtin_fabsf(w) < __builtin_inff())) { ok = false; continue; }
            for (int p = 0; p < k; ++p) ok = ok && selected[(size_t)t * topk + p] != e;
        }
        if (!ok) plan->status = -1;
        else for (int k = 0; k < topk; ++k) atomicAdd(&s_count[selected[(size_t)t * topk + k]], 1);
    }
    __syncthreads();
    for (int e = threadIdx.x; e < n_experts; e += blockDim.x)
        if (s_count[e]) atomicAdd(counts + e, s_count[e]);
}

struct ScanArgs {
    const uint8_t *pool;
    size_t expert_stride;
    int n_experts, hidden, routed;
    int tn_up, tn_down;                  // weight rows per tile of the two matmul launches
    const int *counts;
    int *offsets;                        // [n_experts + 1] row offsets
    int *group_rows;                     // optional copy of the counts for the caller
    PrefillPlan *plan;
    int *status_out;                     // optional
    MfmaJob *gate_up_jobs, *down_jobs;
    const uint16_t *planes_in;  const float *xsum_in;      // split of the inputs, one row per token  [tokens][hidden]
    const uint16_t *planes_act; const float *xsum_act;     // split of the activations, grouped rows   [rows][routed]
    float *gate, *up, *down;
};

// one workgroup: exclusive scans over the experts, job tables for both launches
__global__ __launch_bounds__(MAX_EXPERTS) void group_scan_kernel(const ScanArgs a) {
    __shared__ int s_wave[MAX_EXPERTS / 64];
    const int e = threadIdx.x;
    const int n = e < a.n_experts ? a.counts[e] : 0;
    const int mt = (n + MFMA_TM - 1) / MFMA_TM;
    int rows_total, mt_total, used_total;
    const int row0 = block_exclusive_scan(n, s_wave, &rows_total);
    const int mt0 = block_exclusive_scan(mt, s_wave, &mt_total);
    const int job = block_exclusive_scan(n > 0, s_wave, &used_total);
    if (e < a.n_experts) {
        a.offsets[e] = row0;
        if (a.group_rows) a.group_rows[e] = n;
    }
    const int nt_up = (a.routed + a.tn_up - 1) / a.tn_up, nt_down = (a.hidden + a.tn_down - 1) / a.tn_down;
    const bool valid = a.plan->status == 0;          // written by the previous kernel on this stream
    if (e == 0) {
        a.offsets[a.n_experts] = rows_total;
        a.plan->gate_up_jobs = valid ? 2 * used_total : 0;
        a.plan->down_jobs = valid ? used_total : 0;
        a.plan->gate_up_tiles = valid ? 2 * mt_total * nt_up : 0;
        a.plan->down_tiles = valid ? mt_total * nt_down : 0;
        if (a.status_out) *a.status_out = a.plan->status;
    }
    if (valid && e < a.n_experts && n > 0) {
        const size_t elems = (size_t)a.hidden * (size_t)a.routed;
        const size_t vals_bytes = elems / 2, meta_bytes = (elems / 64) * 2, proj = vals_bytes + 2 * meta_bytes;
        const uint8_t *slot = a.pool + (size_t)e * a.expert_stride;
        for (int p = 0; p < 2; ++p) {
            MfmaJob j;
            j.vals = slot + p * proj; j.scales = j.vals + vals_bytes; j.biases = j.scales + meta_bytes;
            j.planes = a.planes_in;                           // gathered through the row map
            j.xsum = a.xsum_in;
            j.y = (p == 0 ? a.gate : a.up) + (size_t)row0 * a.routed;
            j.tokens = n; j.rows = a.routed;
            j.tile0 = (2 * mt0 + p * mt) * nt_up;
            j.row_base = row0;
            a.gate_up_jobs[2 * job + p] = j;
        }
        MfmaJob d;
        d.vals = slot + 2 * proj; d.scales = d.vals + vals_bytes; d.biases = d.scales + meta_bytes;
        d.planes = a.planes_act + (size_t)row0 * a.routed;
        d.xsum = a.xsum_act + (size_t)row0 * (a.routed >> 6);
        d.y = a.down + (size_t)row0 * a.hidden;
        d.tokens = n; d.rows = a.hidden;
        d.tile0 = mt0 * nt_down;
        d.row_base = 0;
        a.down_jobs[job] = d;
    }
}

// One workgroup of sixteen waves per expert: its (token, rank) pairs in token-major order.  Each wave owns a
// contiguous run of the selection and walks it 64 pairs at a time (one coalesced load), twice: first to count its
// matches, then, knowing how many matches the waves before it hold, to place them.  A match's place inside a chunk
// is the number of matching lanes below it, so the order is the selection's own.
constexpr int FILL_WAVES = 16;

__global__ __launch_bounds__(FILL_WAVES * 64) void group_fill_kernel(const int *__restrict__ selected, int pairs, int topk,
                                                                     const int *__restrict__ offsets, int n_experts,
                                                                     const PrefillPlan *__restrict__ plan,
                                                                     int *__restrict__ row_pairs,
                                                                     int *__restrict__ pair_rows) {
    __shared__ int wave_count[FILL_WAVES];
    if (plan->status != 0) {            // keep the gather in range: every grouped row reads token 0
        for (int p = blockIdx.x * blockDim.x + threadIdx.x; p < pairs; p += gridDim.x * blockDim.x) row_pairs[p] = 0;
        return;
    }
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int e = blockIdx.x;
    if (e >= n_experts || offsets[e + 1] == offsets[e]) return;           // uniform over the workgroup
    const int chunks = (pairs + 63) / 64;
    const int per_wave = (chunks + FILL_WAVES - 1) / FILL_WAVES;
    const int first_chunk = wave * per_wave;
    const int last_chunk = first_chunk + per_wave < chunks ? first_chunk + per_wave : chunks;
    int mine = 0;
    for (int c = first_chunk; c < last_chunk; ++c) {
        const int p = c * 64 + lane;
        mine += __popcll(__ballot(p < pairs && selected[p] == e));
    }
    if (lane == 0) wave_count[wave] = mine;
    __syncthreads();
    int at = offsets[e];
    for (int w = 0; w < wave; ++w) at += wave_count[w];
    for (int c = first_chunk; c < last_chunk; ++c) {
        const int p = c * 64 + lane;
        const bool hit = p < pairs && selected[p] == e;
        const unsigned long long mask = __ballot(hit);
        if (hit) {
            const int row = at + __popcll(mask & ((1ull << lane) - 1ull));
            row_pairs[row] = p;
            pair_rows[p] = row;
        }
        at += __popcll(mask);
    }
}

// out[token][d] = sum over rank of down[row(token, rank)][d] * weight, from +0, rank ascending
__global__ __launch_bounds__(256) void prefill_reduce_kernel(const float *__restrict__ down,
                                                             const int *__restrict__ pair_rows,
                                                             const float *__restrict__ weights, int topk, int hidden,
                                                             const PrefillPlan *__restrict__ plan,
                                                             float *__restrict__ out) {
    if (plan->status != 0) return;
    const int token = blockIdx.x;
    const int d = (blockIdx.y * blockDim.x + threadIdx.x) * 4;            // hidden is a multiple of 64
    if (d >= hidden) return;
    float4 sum = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
    for (int k = 0; k < topk; ++k) {
        const size_t pair = (size_t)token * topk + k;
        const float w = weights[pair];
        const float4 v = *reinterpret_cast<const float4 *>(down + (size_t)pair_rows[pair] * hidden + d);
        float term;
        term = v.x * w; sum.x = sum.x + term;
        term = v.y * w; sum.y = sum.y + term;
        term = v.z * w; sum.z = sum.z + term;
        term = v.w * w; sum.w = sum.w + term;
    }
    *reinterpret_cast<float4 *>(out + (size_t)token * hidden + d) = sum;
}

size_t align256(size_t n) { return (n + 255) & ~(size_t)255; }

struct PrefillWorkspace {
    PrefillPlan *plan; int *counts, *offsets, *pair_rows, *row_pairs;
    MfmaJob *gate_up_jobs, *down_jobs;
    uint16_t *planes_in; float *xsum_in; uint16_t *planes_act; float *xsum_act;
    float *gate, *up, *down;
    size_t bytes;
};

PrefillWorkspace carve(const MoeGeometry &g, int tokens, void *base) {
    PrefillWorkspace w;
    uint8_t *p = (uint8_t *)base;
    const size_t rows = (size_t)tokens * g.topk, E = (size_t)g.n_experts;
    auto take = [&](size_t n) { uint8_t *q = p; p += align256(n); return q; };
    w.plan = (PrefillPlan *)take(sizeof(PrefillPlan));
    w.counts = (int *)take(E * 4);
    w.offsets = (int *)take((E + 1) * 4);
    w.pair_rows = (int *)take(rows * 4);
    w.row_pairs = (int *)take(rows * 4);
    w.gate_up_jobs = (MfmaJob *)take(2 * E * sizeof(MfmaJob));
    w.down_jobs = (MfmaJob *)take(E * sizeof(MfmaJob));
    w.planes_in = (uint16_t *)take(3 * (size_t)tokens * g.hidden * 2);
    w.xsum_in = (float *)take((size_t)tokens * (g.hidden / 64) * 4);
    w.planes_act = (uint16_t *)take(3 * rows * g.routed * 2);
    w.xsum_act = (float *)take(rows * (g.routed / 64) * 4);
    w.gate = (float *)take(rows * g.routed * 4);
    w.up = (float *)take(rows * g.routed * 4);
    w.down = (float *)take(rows * g.hidden * 4);
    w.bytes = (size_t)(p - (uint8_t *)base);
    return w;
}

}  // namespace

size_t moe_prefill_workspace_bytes(const MoeGeometry &g, int tokens) { return carve(g, tokens, nullptr).bytes; }

int moe_prefill_launch(const MoeGeometry &g, const uint8_t *pool, size_t expert_stride, int tokens,
                       const int *selected, const float *weights, const float *inputs, float *outputs,
                       int *group_rows, int *row_pairs, int *status_dev, void *workspace, hipStream_t stream) {
    if (g.n_experts < 1 || g.n_experts > MAX_EXPERTS || g.topk < 1 || g.topk > g.n_experts || tokens < 1 ||
        g.hidden < 64 || (g.hidden & 63) || g.routed < 64 || (g.routed & 63) ||
        (size_t)tokens * (size_t)g.topk > ((size_t)1 << 24))
        return -1;
    const PrefillWorkspace w = carve(g, tokens, workspace);
    const int rows = tokens * g.topk;
    // Tile widths: the wide tile when the upper bound of the grid fills the device twice.
    const int m_upper = rows / MFMA_TM + (g.n_experts < rows ? g.n_experts : rows);
    const int bpw_up = mfma_blocks_per_wave(2LL * m_upper * ((g.routed + 255) / 256));
    const int bpw_down = mfma_blocks_per_wave((long long)m_upper * ((g.hidden + 255) / 256));
    const int tn_up = mfma_tile_rows(bpw_up), tn_down = mfma_tile_rows(bpw_down);
    const int nt_up = (g.routed + tn_up - 1) / tn_up, nt_down = (g.hidden + tn_down - 1) / tn_down;
    // plan and counts are adjacent 256-byte aligned pieces of the workspace: one clear covers both
    static_assert(sizeof(PrefillPlan) <= 256, "the plan fits the first aligned piece");
    if ((uint8_t *)w.counts != (uint8_t *)w.plan + 256) return -1;
    if (clear_words_launch(w.plan, 64 + (size_t)g.n_experts, stream) != 0) return -1;
    hipLaunchKernelGGL(group_count_kernel, dim3((tokens + 255) / 256), dim3(256), 0, stream, selected, weights, tokens,
                       g.topk, g.n_experts, w.counts, w.plan);
    ScanArgs a;
    a.pool = pool; a.expert_stride = expert_stride; a.n_experts = g.n_experts; a.hidden = g.hidden; a.routed = g.routed;
    a.tn_up = tn_up; a.tn_down = tn_down;
    a.counts = w.counts; a.offsets = w.offsets; a.group_rows = group_rows; a.plan = w.plan; a.status_out = status_dev;
    a.gate_up_jobs = w.gate_up_jobs; a.down_jobs = w.down_jobs;
    a.planes_in = w.planes_in; a.xsum_in = w.xsum_in; a.planes_act = w.planes_act; a.xsum_act = w.xsum_act;
    a.gate = w.gate; a.up = w.up; a.down = w.down;
    hipLaunchKernelGGL(group_scan_kernel, dim3(1), dim3(MAX_EXPERTS), 0, stream, a);
    int *rp = row_pairs ? row_pairs : w.row_pairs;
    hipLaunchKernelGGL(group_fill_kernel, dim3(g.n_experts), dim3(FILL_WAVES * 64), 0, stream, selected, rows, g.topk,
                       w.offsets, g.n_experts, w.plan, rp, w.pair_rows);
    if (hipGetLastError() != hipSuccess) return -1;

    // The inputs are split once per token; the matmul gathers the rows of an
    // expert through the row map (pair index / topk = token).  The number of
    // 64-token tiles is known only on the device; the grid covers its upper
    // bound (sum over experts of ceil(n_e / 64) <= rows / 64 + experts) and
    // surplus workgroups leave at once.
    if (x_split_launch(inputs, nullptr, nullptr, 1, g.hidden, tokens, g.hidden, w.planes_in, (size_t)tokens * g.hidden,
                       w.xsum_in, stream) != 0)
        return -1;
    MfmaLaunch gu;
    memset(&gu, 0, sizeof gu);
    gu.table = w.gate_up_jobs; gu.cols = g.hidden; gu.total_tiles = 2 * m_upper * nt_up;
    gu.plane_stride = (size_t)tokens * g.hidden;
    gu.row_map = rp; gu.map_divisor = g.topk; gu.blocks_per_wave = bpw_up;
    gu.njobs_dev = &w.plan->gate_up_jobs; gu.total_tiles_dev = &w.plan->gate_up_tiles;
    if (q4_mfma_launch(gu, stream) != 0) return -1;
    // gelu(gate) * up, split for the down projection
    if (x_split_launch(w.up, w.gate, nullptr, 1, g.routed, rows, g.routed, w.planes_act, (size_t)rows * g.routed,
                       w.xsum_act, stream) != 0)
        return -1;
    MfmaLaunch dn;
    memset(&dn, 0, sizeof dn);
    dn.table = w.down_jobs; dn.cols = g.routed; dn.total_tiles = m_upper * nt_down;
    dn.plane_stride = (size_t)rows * g.routed;
    dn.blocks_per_wave = bpw_down;
    dn.njobs_dev = &w.plan->down_jobs; dn.total_tiles_dev = &w.plan->down_tiles;
    if (q4_mfma_launch(dn, stream) != 0) return -1;
    hipLaunchKernelGGL(prefill_reduce_kernel, dim3(tokens, (g.hidden + 1023) / 1024), dim3(256), 0, stream, w.down,
                       w.pair_rows, weights, g.topk, g.hidden, w.plan, outputs);
    return hipGetLastError() == hipSuccess ? 0 : -1;
}

}  // namespace mi355
