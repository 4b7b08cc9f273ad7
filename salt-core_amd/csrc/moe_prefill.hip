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

// one thread per token: validate and count
__global__ __launch_bounds__(256) void group_count_kernel(const int *__restrict__ selected,
                                                          const float *__restrict__ weights, int tokens, int topk,
                                                          int n_experts, int *__restrict__ counts,
                                                          PrefillPlan *__restrict__ plan) {
    const int t = blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= tokens) return;
    bool ok = true;
    for (int k = 0; k < topk; ++k) {
        const int e = selected[(size_t)t * topk + k];
        const float w = weights[(size_t)t * topk + k];
        if (e < 0 || e >= n_experts || !(__builtin_fabsf(w) < __builtin_inff())) { ok = false; continue; }
        for (int p = 0; p < k; ++p) ok = ok && selected[(size_t)t * topk + p] != e;
    }
    if (!ok) { plan->status = -1; return; }
    for (int k = 0; k < topk; ++k) atomicAdd(counts + selected[(size_t)t * topk + k], 1);
}

struct ScanArgs {
    const uint8_t *pool;
    size_t expert_stride;
    int n_experts, hidden, routed;
    const int *counts;
    int *offsets;                        // [n_experts + 1] row offsets
    int *group_rows;                     // optional copy of the counts for the caller
    PrefillPlan *plan;
    int *status_out;                     // optional
    MfmaJob *gate_up_jobs, *down_jobs;
    const uint16_t *planes_in;  const float *xsum_in;      // split of the gathered inputs  [rows][hidden]
    const uint16_t *planes_act; const float *xsum_act;     // split of the activations      [rows][routed]
    float *gate, *up, *down;
};

// one workgroup: exclusive scans over the experts, job tables for both launches
__global__ __launch_bounds__(MAX_EXPERTS) void group_scan_kernel(const ScanArgs a) {
    __shared__ int s_rows[MAX_EXPERTS], s_mtiles[MAX_EXPERTS], s_used[MAX_EXPERTS];
    const int e = threadIdx.x;
    const int n = e < a.n_experts ? a.counts[e] : 0;
    s_rows[e] = n;
    s_mtiles[e] = (n + MFMA_TM - 1) / MFMA_TM;
    s_used[e] = n > 0;
    __syncthreads();
    int row0 = 0, mt0 = 0, job = 0;
    for (int j = 0; j < e; ++j) { row0 += s_rows[j]; mt0 += s_mtiles[j]; job += s_used[j]; }
    if (e < a.n_experts) {
        a.offsets[e] = row0;
        if (a.group_rows) a.group_rows[e] = n;
    }
    const int nt_up = (a.routed + MFMA_TN - 1) / MFMA_TN, nt_down = (a.hidden + MFMA_TN - 1) / MFMA_TN;
    const bool valid = a.plan->status == 0;          // written by the previous kernel on this stream
    if (e == a.n_experts - 1) {
        a.offsets[a.n_experts] = row0 + n;
        a.plan->gate_up_jobs = valid ? 2 * (job + (n > 0)) : 0;
        a.plan->down_jobs = valid ? job + (n > 0) : 0;
        a.plan->gate_up_tiles = valid ? 2 * (mt0 + s_mtiles[e]) * nt_up : 0;
        a.plan->down_tiles = valid ? (mt0 + s_mtiles[e]) * nt_down : 0;
        if (a.status_out) *a.status_out = a.plan->status;
    }
    if (valid && e < a.n_experts && n > 0) {
        const size_t elems = (size_t)a.hidden * (size_t)a.routed;
        const size_t vals_bytes = elems / 2, meta_bytes = (elems / 64) * 2, proj = vals_bytes + 2 * meta_bytes;
        const uint8_t *slot = a.pool + (size_t)e * a.expert_stride;
        for (int p = 0; p < 2; ++p) {
            MfmaJob j;
            j.vals = slot + p * proj; j.scales = j.vals + vals_bytes; j.biases = j.scales + meta_bytes;
            j.planes = a.planes_in + (size_t)row0 * a.hidden;
            j.xsum = a.xsum_in + (size_t)row0 * (a.hidden >> 6);
            j.y = (p == 0 ? a.gate : a.up) + (size_t)row0 * a.routed;
            j.tokens = n; j.rows = a.routed;
            j.tile0 = (2 * mt0 + p * s_mtiles[e]) * nt_up;
            j.reserved = 0;
            a.gate_up_jobs[2 * job + p] = j;
        }
        MfmaJob d;
        d.vals = slot + 2 * proj; d.scales = d.vals + vals_bytes; d.biases = d.scales + meta_bytes;
        d.planes = a.planes_act + (size_t)row0 * a.routed;
        d.xsum = a.xsum_act + (size_t)row0 * (a.routed >> 6);
        d.y = a.down + (size_t)row0 * a.hidden;
        d.tokens = n; d.rows = a.hidden;
        d.tile0 = mt0 * nt_down;
        d.reserved = 0;
        a.down_jobs[job] = d;
    }
}

// one workgroup per expert: its (token, rank) pairs in token-major order
__global__ __launch_bounds__(256) void group_fill_kernel(const int *__restrict__ selected, int pairs, int topk,
                                                         const int *__restrict__ offsets,
                                                         const PrefillPlan *__restrict__ plan,
                                                         int *__restrict__ row_pairs, int *__restrict__ pair_rows) {
    __shared__ int s_wave[4];
    __shared__ int s_base;
    if (plan->status != 0) {            // keep the gather in range: every grouped row reads token 0
        for (int p = blockIdx.x * 256 + threadIdx.x; p < pairs; p += gridDim.x * 256) row_pairs[p] = 0;
        return;
    }
    const int e = blockIdx.x;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    if (threadIdx.x == 0) s_base = offsets[e];
    __syncthreads();
    for (int first = 0; first < pairs; first += 256) {
        const int p = first + threadIdx.x;
        const bool hit = p < pairs && selected[p] == e;
        const unsigned long long mask = __ballot(hit);
        const int before = __popcll(mask & ((1ull << lane) - 1ull));
        if (lane == 0) s_wave[wave] = __popcll(mask);
        __syncthreads();
        int base = s_base;
        for (int w = 0; w < wave; ++w) base += s_wave[w];
        if (hit) { row_pairs[base + before] = p; pair_rows[p] = base + before; }
        __syncthreads();
        if (threadIdx.x == 0) s_base += s_wave[0] + s_wave[1] + s_wave[2] + s_wave[3];
        __syncthreads();
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
    const int d = blockIdx.y * blockDim.x + threadIdx.x;
    if (d >= hidden) return;
    float sum = 0.0f;
    for (int k = 0; k < topk; ++k) {
        const size_t pair = (size_t)token * topk + k;
        const float term = down[(size_t)pair_rows[pair] * hidden + d] * weights[pair];
        sum = sum + term;
    }
    out[(size_t)token * hidden + d] = sum;
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
    w.planes_in = (uint16_t *)take(3 * rows * g.hidden * 2);
    w.xsum_in = (float *)take(rows * (g.hidden / 64) * 4);
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
    const int nt_up = (g.routed + MFMA_TN - 1) / MFMA_TN, nt_down = (g.hidden + MFMA_TN - 1) / MFMA_TN;
    if (hipMemsetAsync(w.plan, 0, sizeof(PrefillPlan), stream) != hipSuccess ||
        hipMemsetAsync(w.counts, 0, (size_t)g.n_experts * 4, stream) != hipSuccess)
        return -1;
    hipLaunchKernelGGL(group_count_kernel, dim3((tokens + 255) / 256), dim3(256), 0, stream, selected, weights, tokens,
                       g.topk, g.n_experts, w.counts, w.plan);
    ScanArgs a;
    a.pool = pool; a.expert_stride = expert_stride; a.n_experts = g.n_experts; a.hidden = g.hidden; a.routed = g.routed;
    a.counts = w.counts; a.offsets = w.offsets; a.group_rows = group_rows; a.plan = w.plan; a.status_out = status_dev;
    a.gate_up_jobs = w.gate_up_jobs; a.down_jobs = w.down_jobs;
    a.planes_in = w.planes_in; a.xsum_in = w.xsum_in; a.planes_act = w.planes_act; a.xsum_act = w.xsum_act;
    a.gate = w.gate; a.up = w.up; a.down = w.down;
    hipLaunchKernelGGL(group_scan_kernel, dim3(1), dim3(MAX_EXPERTS), 0, stream, a);
    int *rp = row_pairs ? row_pairs : w.row_pairs;
    hipLaunchKernelGGL(group_fill_kernel, dim3(g.n_experts), dim3(256), 0, stream, selected, rows, g.topk, w.offsets,
                       w.plan, rp, w.pair_rows);
    if (hipGetLastError() != hipSuccess) return -1;

    // gather + split: grouped row r reads token row_pairs[r] / topk
    if (x_split_launch(inputs, nullptr, rp, g.topk, g.hidden, rows, g.hidden, w.planes_in, (size_t)rows * g.hidden,
                       w.xsum_in, stream) != 0)
        return -1;
    // The number of 64-token tiles is known only on the device; the grid covers
    // its upper bound (sum over experts of ceil(n_e / TM) <= rows / TM + experts)
    // and surplus workgroups leave at once.
    const int m_upper = rows / MFMA_TM + (g.n_experts < rows ? g.n_experts : rows);
    MfmaLaunch gu;
    memset(&gu, 0, sizeof gu);
    gu.table = w.gate_up_jobs; gu.cols = g.hidden; gu.total_tiles = 2 * m_upper * nt_up;
    gu.plane_stride = (size_t)rows * g.hidden;
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
    dn.njobs_dev = &w.plan->down_jobs; dn.total_tiles_dev = &w.plan->down_tiles;
    if (q4_mfma_launch(dn, stream) != 0) return -1;
    hipLaunchKernelGGL(prefill_reduce_kernel, dim3(tokens, (g.hidden + 255) / 256), dim3(256), 0, stream, w.down,
                       w.pair_rows, weights, g.topk, g.hidden, w.plan, outputs);
    return hipGetLastError() == hipSuccess ? 0 : -1;
}

}  // namespace mi355
