// Router top-k, GELU gating and the ordered expert reduction of the MoE decode
// layer-step, and the launch sequence that strings them together with the
// affine-Q4 expert projections.
//
// reference models/gemma4-26b-a4b/src/gemma4.c:132-186 (router top-k),
//           gemma4_text.c:7923-7930 (ascending sort of the selection),
//           gemma4_text.c:7608-7649 (expert: gate, up, gelu*up, down),
//           gemma4_text.c:8301-8304 (weighted sum in ascending expert order).
//
// The router's insertion list is the stable descending order of the logits
// (a later expert must be strictly greater to pass an earlier one), so an
// expert's position is its rank: the number of larger logits plus the number
// of equal logits with a smaller index.  Ranks are computed in parallel; the
// two fp32 sums whose order the reference fixes (over all experts ascending,
// over the selected experts in list order) are done by one lane, in order.
#include "device_math.h"
#include "mi355_internal.h"
#include "router_device.h"

#include <string.h>

namespace mi355 {
namespace {

struct JobEmit {                 // where the router kernel writes the step's Q4 job tables (may be all-null)
    Q4Job *gate_up_jobs;
    Q4Job *down_jobs;
    const uint8_t *pool;
    size_t expert_stride;
    const float *x;
    float *gate, *up, *act, *expert_out;
    int hidden, routed;
};

__global__ __launch_bounds__(ROUTER_MAX_EXPERTS) void router_topk_kernel(
        const float *__restrict__ logits, const float *__restrict__ per_expert_scale, int n_experts, int topk,
        int sorted_by_id, int *__restrict__ selected, float *__restrict__ weights, int *__restrict__ status,
        JobEmit emit) {
    __shared__ RouterShared sh;
    router_topk_block(logits, per_expert_scale, n_experts, topk, sorted_by_id != 0, true, sh);
    const int e = threadIdx.x;
    const int bad = sh.bad;
    if (e == 0) *status = bad ? -1 : 0;
    if (e < topk) {
        const int place = e;
        const int expert = sh.out_sel[place];
        if (!bad) {                              // a rejected call leaves the caller's outputs untouched
            selected[place] = expert;
            weights[place] = sh.out_w[place];
        }
        if (emit.gate_up_jobs) {
            const size_t n = (size_t)emit.hidden * (size_t)emit.routed;
            const size_t vals_bytes = n / 2, meta_bytes = (n / 64) * 2;
            const size_t proj_bytes = vals_bytes + 2 * meta_bytes;
            const uint8_t *slot = emit.pool + (size_t)expert * emit.expert_stride;
            const int up_tiles = (emit.routed + 63) / 64, down_tiles = (emit.hidden + 63) / 64;
            for (int p = 0; p < 2; ++p) {
                Q4Job job;
                job.vals = slot + p * proj_bytes;
                job.scales = job.vals + vals_bytes;
                job.biases = job.scales + meta_bytes;
                job.x = emit.x;
                job.y = (p == 0 ? emit.gate : emit.up) + (size_t)place * emit.routed;
                job.rows = emit.routed;
                job.tile0 = (2 * place + p) * up_tiles;
                job.x_stride = emit.hidden;
                job.y_stride = emit.routed;
                emit.gate_up_jobs[2 * place + p] = job;
            }
            Q4Job down;
            down.vals = slot + 2 * proj_bytes;
            down.scales = down.vals + vals_bytes;
            down.biases = down.scales + meta_bytes;
            down.x = emit.act + (size_t)place * emit.routed;
            down.y = emit.expert_out + (size_t)place * emit.hidden;
            down.rows = emit.hidden;
            down.tile0 = place * down_tiles;
            down.x_stride = emit.routed;
            down.y_stride = emit.hidden;
            emit.down_jobs[place] = down;
        }
    }
}

__global__ __launch_bounds__(256) void moe_activate_kernel(const float *__restrict__ gate,
                                                           const float *__restrict__ up, float *__restrict__ act,
                                                           size_t n) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) act[i] = det_gelu_tanh(gate[i]) * up[i];
}

__global__ __launch_bounds__(256) void moe_reduce_kernel(const float *__restrict__ expert_out,
                                                         const float *__restrict__ weights, int topk, int hidden,
                                                         const int *__restrict__ status, float *__restrict__ out) {
    if (status && *status != 0) return;          // the router rejected its input: nothing was computed
    const int d = blockIdx.x * blockDim.x + threadIdx.x;
    if (d >= hidden) return;
    float sum = 0.0f;
    for (int i = 0; i < topk; ++i) {
        const float term = expert_out[(size_t)i * hidden + d] * weights[i];
        sum = sum + term;
    }
    out[d] = sum;
}

size_t align256(size_t n) { return (n + 255) & ~(size_t)255; }

}  // namespace

size_t moe_workspace_bytes(const MoeGeometry &g) {
    const size_t k = (size_t)g.topk;
    return align256(256) + align256(2 * k * sizeof(Q4Job)) + align256(k * sizeof(Q4Job)) +
           3 * align256(k * g.routed * sizeof(float)) + align256(k * g.hidden * sizeof(float)) +
           align256((size_t)((g.hidden + 63) / 64) * sizeof(int));
}

void moe_workspace_carve(const MoeGeometry &g, void *base, MoeWorkspace *ws) {
    uint8_t *p = (uint8_t *)base;
    const size_t k = (size_t)g.topk;
    ws->status = (int *)p;                  p += align256(256);
    ws->gate_up_jobs = (Q4Job *)p;          p += align256(2 * k * sizeof(Q4Job));
    ws->down_jobs = (Q4Job *)p;             p += align256(k * sizeof(Q4Job));
    ws->gate = (float *)p;                  p += align256(k * g.routed * sizeof(float));
    ws->up = (float *)p;                    p += align256(k * g.routed * sizeof(float));
    ws->act = (float *)p;                   p += align256(k * g.routed * sizeof(float));
    ws->expert_out = (float *)p;            p += align256(k * g.hidden * sizeof(float));
    ws->arrivals = (int *)p;
}

int router_topk_launch(const float *logits, const float *per_expert_scale, int n_experts, int topk,
                       int sorted_by_id, int *selected, float *weights, int *status, hipStream_t stream) {
    if (n_experts < 1 || n_experts > ROUTER_MAX_EXPERTS || topk < 1 || topk > n_experts || topk > ROUTER_MAX_TOPK)
        return -1;
    JobEmit none = {};
    const int threads = ((n_experts > topk ? n_experts : topk) + 63) & ~63;
    hipLaunchKernelGGL(router_topk_kernel, dim3(1), dim3(threads), 0, stream, logits, per_expert_scale, n_experts,
                       topk, sorted_by_id, selected, weights, status, none);
    return hipGetLastError() == hipSuccess ? 0 : -1;
}

int moe_activate_launch(const float *gate, const float *up, float *act, size_t n, hipStream_t stream) {
    hipLaunchKernelGGL(moe_activate_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, stream, gate, up, act, n);
    return hipGetLastError() == hipSuccess ? 0 : -1;
}

int moe_reduce_launch(const float *expert_out, const float *weights, int topk, int hidden, float *out,
                      const int *status, hipStream_t stream) {
    hipLaunchKernelGGL(moe_reduce_kernel, dim3((hidden + 255) / 256), dim3(256), 0, stream, expert_out, weights, topk,
                       hidden, status, out);
    return hipGetLastError() == hipSuccess ? 0 : -1;
}

int moe_decode_step_launch(const MoeGeometry &g, const uint8_t *pool, size_t expert_stride, const float *logits,
                           const float *per_expert_scale, const float *x, int *selected, float *weights,
                           float *expert_out, float *out, const MoeWorkspace &ws, float code_scale,
                           hipStream_t stream) {
    if (g.n_experts < 1 || g.n_experts > ROUTER_MAX_EXPERTS || g.topk < 1 || g.topk > g.n_experts ||
        g.topk > ROUTER_MAX_TOPK || g.hidden < 64 || (g.hidden & 63) || g.routed < 64 || (g.routed & 63))
        return -1;
    float *eo = expert_out ? expert_out : ws.expert_out;
    if (g.n_experts <= MOE_FUSE_MAX_EXPERTS && g.routed <= MOE_FUSE_MAX_ROUTED) {
        // Two launches: router + gate/up, then activation + down + the ordered reduction (by the last workgroup
        // to finish each tile of the output).
        Q4Launch fused;
        memset(&fused, 0, sizeof fused);
        fused.code_scale = code_scale;
        MoeFuse &m = fused.moe;
        m.logits = logits; m.per_expert_scale = per_expert_scale; m.pool = pool; m.expert_stride = expert_stride;
        m.x = x; m.gate = ws.gate; m.up = ws.up; m.expert_out = eo; m.selected = selected; m.weights = weights;
        m.status = ws.status; m.n_experts = g.n_experts; m.topk = g.topk; m.hidden = g.hidden; m.routed = g.routed;
        m.out = out; m.arrivals = out ? ws.arrivals : nullptr;
        if (q4_moe_gate_up_launch(fused, stream) != 0) return -1;
        return q4_moe_down_launch(fused, stream);
    }
    JobEmit emit;
    emit.gate_up_jobs = ws.gate_up_jobs;
    emit.down_jobs = ws.down_jobs;
    emit.pool = pool;
    emit.expert_stride = expert_stride;
    emit.x = x;
    emit.gate = ws.gate; emit.up = ws.up; emit.act = ws.act; emit.expert_out = eo;
    emit.hidden = g.hidden; emit.routed = g.routed;
    const int threads = (g.n_experts + 63) & ~63;
    hipLaunchKernelGGL(router_topk_kernel, dim3(1), dim3(threads), 0, stream, logits, per_expert_scale, g.n_experts,
                       g.topk, 1, selected, weights, ws.status, emit);
    if (hipGetLastError() != hipSuccess) return -1;

    Q4Launch gate_up;
    memset(&gate_up, 0, sizeof gate_up);
    gate_up.table = ws.gate_up_jobs;
    gate_up.njobs = 2 * g.topk;
    gate_up.cols = g.hidden;
    gate_up.tokens = 1;
    gate_up.total_tiles = 2 * g.topk * ((g.routed + 63) / 64);
    gate_up.code_scale = code_scale;
    if (q4_launch(gate_up, 0, stream) != 0) return -1;

    if (moe_activate_launch(ws.gate, ws.up, ws.act, (size_t)g.topk * g.routed, stream) != 0) return -1;

    Q4Launch down;
    memset(&down, 0, sizeof down);
    down.table = ws.down_jobs;
    down.njobs = g.topk;
    down.cols = g.routed;
    down.tokens = 1;
    down.total_tiles = g.topk * ((g.hidden + 63) / 64);
    down.code_scale = code_scale;
    if (q4_launch(down, 0, stream) != 0) return -1;

    return out ? moe_reduce_launch(eo, weights, g.topk, g.hidden, out, nullptr, stream) : 0;
}

// The same step on the tolerance-class matvec kernels: router top-k (bit-exact), gate and up, gelu_tanh(gate) * up,
// down, ordered weighted sum.  Two launches where moe_dot16.hip serves the geometry (the activation rides in the
// first, the weighted sum in the second), else three launches on the 32-row kernel with the sum on its own.
// Returns 0, MOE16_NOT_SERVED when neither plan takes the geometry (nothing was launched), or -1 when a launch failed.
int moe_decode_step_t_launch(const MoeGeometry &g, const uint8_t *pool, size_t expert_stride, const float *logits,
                             const float *per_expert_scale, const float *x, int *selected, float *weights,
                             float *expert_out, float *out, const MoeWorkspace &ws, hipStream_t stream) {
    MoeFuse m;
    memset(&m, 0, sizeof m);
    m.logits = logits; m.per_expert_scale = per_expert_scale; m.pool = pool; m.expert_stride = expert_stride;
    m.x = x; m.gate = ws.gate; m.up = ws.up; m.expert_out = expert_out ? expert_out : ws.expert_out;
    m.selected = selected; m.weights = weights; m.status = ws.status;
    m.n_experts = g.n_experts; m.topk = g.topk; m.hidden = g.hidden; m.routed = g.routed;
    m.act = ws.act;
    if (out) {
        MoeFuse two = m;
        two.expert_out = expert_out;              // optional there
        const int served = moe16_step_launch(two, out, stream);
        if (served == 0) return 0;
        if (served != MOE16_NOT_SERVED) return -1;    // a launch failed: nothing to fall back on
    }
    if (!q4_dot_moe_serves(m)) return MOE16_NOT_SERVED;   // nothing launched: the caller takes the bit-exact plan
    if (q4_dot_moe_gate_up_launch(m, stream) != 0) return -1;
    if (q4_dot_moe_down_launch(m, stream) != 0) return -1;
    return out ? moe_reduce_launch(m.expert_out, weights, g.topk, g.hidden, out, ws.status, stream) : 0;
}

}  // namespace mi355
