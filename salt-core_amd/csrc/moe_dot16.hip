// The MoE decode layer-step (reference gemma4_text.c:8360, 7923-7930, 7608-7649, 8301-8304) in two launches on the
// sixteen-row tolerance-class stream (q4_dot16_core.h):
//
//  1. gate, up and the activation.  A workgroup owns 16 rows of one selected expert's gate AND up projection: waves
//     2p and 2p + 1 walk part p of the steps of the gate and the up matrix, the parts meet in LDS in part order and
//     wave 0 writes act = gelu_tanh(gate) * up.  Every wave finds its expert with the wave-level router search; one
//     workgroup past the tiles runs the whole router and publishes selection, weights and status (bit-exact).
//  2. down and the ordered weighted sum.  A workgroup owns 16 rows of the layer output: wave e walks the down
//     projection of the e-th selected expert over that expert's activation (the digit planes of all selected experts
//     are built once per workgroup), the expert outputs meet in LDS and wave 0 adds them in ascending expert order,
//     every product and every sum rounded separately as the reference does.  No launch for the activation, none for
//     the sum, no traffic between workgroups.
#include "q4_dot16_core.h"
#include "device_math.h"
#include "router_device.h"

#include <stdio.h>
#include <string.h>

namespace mi355 {
namespace {

constexpr int MOE16_MAX_TOPK = 8;            // waves of the second launch

template <int PARTS, int MD>
__global__ __launch_bounds__(2 * PARTS * 64) void moe16_gate_up_kernel(const MoeFuse m, int blocks_per_place) {
    constexpr int WAVES = 2 * PARTS, THREADS = WAVES * 64;
    static_assert(sizeof(RouterShared) <= (size_t)WAVES * WAVE16_LDS, "the publishing workgroup borrows the weight staging memory");
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int tiles = m.topk * blocks_per_place;

    if ((int)blockIdx.x == tiles) {                  // the publisher: the whole router, ordered sums and all
        RouterShared &sh = *reinterpret_cast<RouterShared *>(lds);
        router_topk_block(m.logits, m.per_expert_scale, m.n_experts, m.topk, true, true, sh);
        const int bad = sh.bad;
        if (tid == 0) *m.status = bad ? -1 : 0;
        if (tid < m.topk && !bad) { m.selected[tid] = sh.out_sel[tid]; m.weights[tid] = sh.out_w[tid]; }
        return;
    }
    Dot16Stream<MD> stream;
    stream.setup(lane, m.hidden, lds + (size_t)wave * WAVE16_LDS);
    const int SG = stream.SG;
    uint8_t *const zero_lds = lds + WAVES * WAVE16_LDS;
    uint8_t *const img_lds = zero_lds + ZERO_BYTES;
    float *const xm_lds = (float *)(img_lds + (size_t)2 * SG * GROUP_IMAGE);

    const int place = (int)blockIdx.x / blocks_per_place, block = (int)blockIdx.x - place * blocks_per_place;
    // The activation and the router's inputs are requested together, the activation first: when the logits have
    // arrived, so has the activation, and the weight loads that follow queue behind neither.
    const ImageItems items(1, stream.ngrp);
    Q4ImageBuilder<THREADS> image;
    image.request_early(tid, items, [&](int) { return m.x; });
    // every wave finds its expert on its own (with finite inputs the router cannot fail later) and sends for its
    // scales and first weights at once: they are on their way while the digit planes are built
    const int expert = router_select_wave(m.logits, m.per_expert_scale, m.n_experts, m.topk, place);
    image.settle(expert, items);
    if (expert < 0) return;                          // uniform: every wave sees the same inputs; no barrier passed yet
    const size_t n_weights = (size_t)m.hidden * (size_t)m.routed;
    const size_t vals_bytes = n_weights / 2, meta_bytes = (n_weights / 64) * 2, proj_bytes = vals_bytes + 2 * meta_bytes;
    const int which = wave & 1, part = wave >> 1;    // 0 gate, 1 up
    const uint8_t *vals = m.pool + (size_t)expert * m.expert_stride + (size_t)which * proj_bytes;
    const int row_base = block * ROWS16;
    stream.bind(vals, vals + vals_bytes, vals + vals_bytes + meta_bytes, m.routed, row_base,
                part * stream.nstage / PARTS, (part + 1) * stream.nstage / PARTS);
    stream.start();
    image.build(tid, items, SG, zero_lds, img_lds, xm_lds, [&](int, size_t column, float (&xv)[8]) {
#pragma unroll
        for (int k = 0; k < 8; ++k) xv[k] = m.x[column + k];
    });
    __syncthreads();                                 // the digit planes are in place

    Dot16Operand operand[1] = {dot16_operand(lane, 0, true, 0, 0, SG, zero_lds, img_lds, xm_lds)};
    float acc[1] = {0.0f};
    stream.run(operand, acc);

    // the strips meet in the wave, the parts and the two matrices in LDS (the wave's own staging memory is idle now)
    const float sum = acc[0] + __shfl_xor(acc[0], 16, 64);
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
    if (lane < 16) ((float *)stream.my_lds)[lane] = sum;
    __syncthreads();
    if (wave == 0 && lane < stream.rows_here && lane < 16) {
        float gate = 0.0f, up = 0.0f;
        for (int p = 0; p < PARTS; ++p) {
            gate = gate + ((const float *)(lds + (size_t)(2 * p) * WAVE16_LDS))[lane];
            up = up + ((const float *)(lds + (size_t)(2 * p + 1) * WAVE16_LDS))[lane];
        }
        m.act[(size_t)place * m.routed + row_base + lane] = det_gelu_tanh(gate) * up;
    }
}

template <int MD>
__global__ __launch_bounds__(MOE16_MAX_TOPK * 64) void moe16_down_sum_kernel(const MoeFuse m, float *out) {
    constexpr int WAVES = MOE16_MAX_TOPK, THREADS = WAVES * 64;
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    Dot16Stream<MD> stream;
    stream.setup(lane, m.routed, lds + (size_t)wave * WAVE16_LDS);
    const int SG = stream.SG;
    // The activations of all selected experts (expert e of the selection is "token" e of the digit planes) are
    // requested first, together with the status and the selection, and the weight loads go out when they have
    // arrived: the digit planes are then built while the weights are on their way (weights first, activations
    // queued behind them, cost the step a microsecond).  A rejected step leaves whatever an earlier step wrote in
    // the activations; it is fetched and dropped.
    const int topk = m.topk;
    const ImageItems items(topk, stream.ngrp);
    Q4ImageBuilder<THREADS> image;
    image.request_early(tid, items, [&](int e) { return m.act + (size_t)e * m.routed; });
    // what the first launch left: status, selection and routing weights, fetched in one go as wave-uniform values
    typedef const int __attribute__((address_space(4))) *uniform_int_ptr;
    typedef const float __attribute__((address_space(4))) *uniform_float_ptr;
    const bool has_expert = wave < topk;
    const int status = *(uniform_int_ptr)(uintptr_t)m.status;
    const int expert = ((uniform_int_ptr)(uintptr_t)m.selected)[has_expert ? wave : 0];
    float routing[WAVES];
#pragma unroll
    for (int e = 0; e < WAVES; ++e) routing[e] = ((uniform_float_ptr)(uintptr_t)m.weights)[e < topk ? e : 0];
    if (status != 0) {                               // the router rejected its input
        image.settle(status, items);                 // nothing of the wave's may be in flight when it ends
        return;
    }
    uint8_t *const zero_lds = lds + WAVES * WAVE16_LDS;
    uint8_t *const img_lds = zero_lds + ZERO_BYTES;                        // [expert of the selection][2 * SG][GROUP_IMAGE]
    float *const xm_lds = (float *)(img_lds + (size_t)WAVES * 2 * SG * GROUP_IMAGE);

    const int row_base = (int)blockIdx.x * ROWS16;
    const size_t n_weights = (size_t)m.hidden * (size_t)m.routed;
    const size_t vals_bytes = n_weights / 2, meta_bytes = (n_weights / 64) * 2, proj_bytes = vals_bytes + 2 * meta_bytes;
    image.settle(expert, items);
    if (has_expert) {
        const uint8_t *vals = m.pool + (size_t)expert * m.expert_stride + 2 * proj_bytes;
        stream.bind(vals, vals + vals_bytes, vals + vals_bytes + meta_bytes, m.hidden, row_base, 0, stream.nstage);
        stream.start();
    }
    image.build(tid, items, SG, zero_lds, img_lds, xm_lds, [&](int e, size_t column, float (&xv)[8]) {
#pragma unroll
        for (int k = 0; k < 8; ++k) xv[k] = m.act[(size_t)e * m.routed + column + k];
    });
    __syncthreads();

    float sum = 0.0f;
    if (has_expert) {
        Dot16Operand operand[1] = {dot16_operand(lane, 0, true, wave, wave, SG, zero_lds, img_lds, xm_lds)};
        float acc[1] = {0.0f};
        stream.run(operand, acc);
        sum = acc[0] + __shfl_xor(acc[0], 16, 64);
        if (m.expert_out && lane < 16 && lane < stream.rows_here) m.expert_out[(size_t)wave * m.hidden + row_base + lane] = sum;
    }
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
    if (lane < 16) ((float *)(lds + (size_t)wave * WAVE16_LDS))[lane] = sum;
    __syncthreads();
    const int rows_here = m.hidden - row_base < ROWS16 ? m.hidden - row_base : ROWS16;
    if (wave == 0 && lane < rows_here && lane < 16) {
        // reference gemma4_text.c:8301-8304: out = 0; out += o_i * w_i in ascending expert order, product and sum
        // rounded separately
        float total = 0.0f;
#pragma unroll
        for (int e = 0; e < WAVES; ++e) {
            if (e < topk) {
                const float term = ((const float *)(lds + (size_t)e * WAVE16_LDS))[lane] * routing[e];
                total = total + term;
            }
        }
        out[row_base + lane] = total;
    }
}

size_t moe16_gate_up_lds(int hidden, int waves) {
    const int sg = dot_steps(hidden >> 6) * STAGE_GROUPS;
    return (size_t)waves * WAVE16_LDS + ZERO_BYTES + (size_t)2 * sg * (GROUP_IMAGE + 8);
}
size_t moe16_down_lds(int routed) {
    const int sg = dot_steps(routed >> 6) * STAGE_GROUPS;
    return (size_t)MOE16_MAX_TOPK * WAVE16_LDS + ZERO_BYTES + (size_t)MOE16_MAX_TOPK * 2 * sg * (GROUP_IMAGE + 8);
}

template <class Kernel>
int raise_lds(Kernel kernel, size_t lds, size_t &raised) {
    if (lds <= raised) return 0;
    if (hipFuncSetAttribute((const void *)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess) return -1;
    raised = lds;
    return 0;
}

template <int PARTS, int MD>
int launch_gate_up(const MoeFuse &m, int blocks, size_t lds, hipStream_t stream) {
    static size_t raised = 0;
    if (raise_lds(moe16_gate_up_kernel<PARTS, MD>, lds, raised) != 0) return -1;
    hipLaunchKernelGGL((moe16_gate_up_kernel<PARTS, MD>), dim3(m.topk * blocks + 1), dim3(2 * PARTS * 64), lds, stream, m, blocks);
    return hipGetLastError() == hipSuccess ? 0 : -1;
}

template <int MD>
int launch_down_sum(const MoeFuse &m, float *out, size_t lds, hipStream_t stream) {
    static size_t raised = 0;
    if (raise_lds(moe16_down_sum_kernel<MD>, lds, raised) != 0) return -1;
    hipLaunchKernelGGL((moe16_down_sum_kernel<MD>), dim3((m.hidden + ROWS16 - 1) / ROWS16), dim3(MOE16_MAX_TOPK * 64), lds,
                       stream, m, out);
    return hipGetLastError() == hipSuccess ? 0 : -1;
}

// dwords of scales a lane keeps for a wave that walks `steps` steps of a strip: two groups per dword
int meta_dwords(int steps) { return steps <= 2 ? 4 : steps <= 4 ? 8 : 16; }

}  // namespace

// 0: both launches are enqueued.  MOE16_NOT_SERVED: this geometry is not served, nothing was launched (the caller
// takes another plan).  -1: a launch failed.
int moe16_step_launch(const MoeFuse &m, float *out, hipStream_t stream) {
    if (m.n_experts < 1 || m.n_experts > ROUTER_WAVE_MAX_EXPERTS || m.topk < 1 || m.topk > MOE16_MAX_TOPK ||
        m.topk > m.n_experts || !q4_dot_takes(m.hidden) || !q4_dot_takes(m.routed) || !out || !m.act)
        return MOE16_NOT_SERVED;
    const int steps_hidden = dot_steps(m.hidden >> 6), steps_routed = dot_steps(m.routed >> 6);
    // three parts per matrix where the row has at least three steps, else one
    const int parts = steps_hidden >= 3 ? 3 : 1;
    const int steps_a = (steps_hidden + parts - 1) / parts;
    if (steps_a > 8 || steps_routed > 8) return MOE16_NOT_SERVED;   // a lane's registers hold the scales of at most 32 groups
    if (m.n_experts > 2 * parts * 64) return MOE16_NOT_SERVED;      // the publishing workgroup runs the router with one thread per expert
    const size_t lds_a = moe16_gate_up_lds(m.hidden, 2 * parts), lds_b = moe16_down_lds(m.routed);
    if (lds_a > DOT_LDS_LIMIT || lds_b > DOT_LDS_LIMIT) return MOE16_NOT_SERVED;
    const int blocks = (m.routed + ROWS16 - 1) / ROWS16;
    const int md_a = meta_dwords(steps_a), md_b = meta_dwords(steps_routed);
    int rc;
    if (parts == 3)
        rc = md_a == 4 ? launch_gate_up<3, 4>(m, blocks, lds_a, stream)
           : md_a == 8 ? launch_gate_up<3, 8>(m, blocks, lds_a, stream) : launch_gate_up<3, 16>(m, blocks, lds_a, stream);
    else
        rc = md_a == 4 ? launch_gate_up<1, 4>(m, blocks, lds_a, stream)
           : md_a == 8 ? launch_gate_up<1, 8>(m, blocks, lds_a, stream) : launch_gate_up<1, 16>(m, blocks, lds_a, stream);
    if (rc != 0) return -1;
    rc = md_b == 4 ? launch_down_sum<4>(m, out, lds_b, stream)
       : md_b == 8 ? launch_down_sum<8>(m, out, lds_b, stream) : launch_down_sum<16>(m, out, lds_b, stream);
    note_kernel("moe16_gate_up_kernel<%d,%d> + moe16_down_sum_kernel<%d>", parts, md_a, md_b);
    return rc;
}

}  // namespace mi355
