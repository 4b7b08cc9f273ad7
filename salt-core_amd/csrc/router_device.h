// Router top-k of one workgroup (reference models/gemma4-26b-a4b/src/gemma4.c:132-186,
// ascending sort gemma4_text.c:7923-7930), shared by the stand-alone router
// kernel and by the prologue of the fused gate/up launch.
//
// The reference's insertion list is the stable descending order of the logits
// (a later expert must be strictly greater to pass an earlier one), so an
// expert's position is its rank: the number of larger logits plus the number
// of equal logits with a smaller index.  Ranks are computed in parallel; the
// two fp32 sums whose order the reference fixes (over all experts ascending,
// over the selected experts in list order) are done by one lane, in order.
#pragma once

#include "device_math.h"

#include <hip/hip_runtime.h>

namespace mi355 {

constexpr int ROUTER_MAX_EXPERTS = 1024;
constexpr int ROUTER_MAX_TOPK = 64;

struct RouterShared {
    float logit[ROUTER_MAX_EXPERTS];
    float expv[ROUTER_MAX_EXPERTS];
    float wave_max[ROUTER_MAX_EXPERTS / 64];
    int rank[ROUTER_MAX_EXPERTS];
    int sel[ROUTER_MAX_TOPK];          // list order (descending logit)
    float w[ROUTER_MAX_TOPK];
    int out_sel[ROUTER_MAX_TOPK];      // output order: list order, or ascending expert id
    float out_w[ROUTER_MAX_TOPK];
    int bad;
    float peak;
};

// Every thread of the workgroup calls this; blockDim.x is a multiple of 64 and
// at least max(n_experts, topk).  On return (after its last barrier) sh.bad
// tells whether an input was non-finite, sh.out_sel[0..topk) holds the chosen
// experts and, when want_weights, sh.out_w their weights.  With finite inputs
// the two sums cannot fail (the largest term of the first is exp(0) = 1 and its
// expert is always chosen), so a caller that only needs the selection may skip
// the weights and still learn every rejection.
__device__ __forceinline__ void router_topk_block(const float *__restrict__ logits,
                                                  const float *__restrict__ per_expert_scale, int n_experts, int topk,
                                                  bool sorted_by_id, bool want_weights, RouterShared &sh) {
    const int e = threadIdx.x;
    const bool live = e < n_experts;
    if (e == 0) sh.bad = 0;
    __syncthreads();
    float mine = -__builtin_inff();
    if (live) {
        mine = logits[e];
        const float sc = per_expert_scale[e];
        if (!(__builtin_fabsf(mine) < __builtin_inff()) || !(__builtin_fabsf(sc) < __builtin_inff())) sh.bad = 1;
        sh.logit[e] = mine;
    }
    // max over finite values is exact in any order
    float m = mine;
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) m = fmaxf(m, __shfl_xor(m, off, 64));
    if ((e & 63) == 0 && e < ROUTER_MAX_EXPERTS) sh.wave_max[e >> 6] = m;
    __syncthreads();
    int bad = sh.bad;
    if (e == 0) {
        float peak = sh.wave_max[0];
        const int waves = (n_experts + 63) >> 6;
        for (int w = 1; w < waves; ++w) peak = fmaxf(peak, sh.wave_max[w]);
        sh.peak = peak;
    }
    __syncthreads();
    const float peak = sh.peak;
    // Ranks: the comparisons of one expert are spread over as many threads as
    // the workgroup has to spare (integer counts, so the split changes nothing).
    const int padded = (n_experts + 63) & ~63;
    const int parts = (int)blockDim.x / padded > 0 ? (int)blockDim.x / padded : 1;
    if (live) sh.rank[e] = 0;
    __syncthreads();
    if (!bad && e < padded * parts) {
        const int who = e % padded, part = e / padded;
        if (who < n_experts) {
            const float self = sh.logit[who];
            const int span = (n_experts + parts - 1) / parts;
            const int first = part * span, last = first + span < n_experts ? first + span : n_experts;
            int count = 0;
            for (int j = first; j < last; ++j) {
                const float other = sh.logit[j];
                count += (other > self) || (other == self && j < who);
            }
            if (parts > 1) atomicAdd(&sh.rank[who], count); else sh.rank[who] = count;
        }
    }
    __syncthreads();
    if (!bad && live) {
        if (want_weights) sh.expv[e] = det_expf(mine - peak);
        if (sh.rank[e] < topk) sh.sel[sh.rank[e]] = e;
    }
    __syncthreads();
    if (want_weights && e == 0 && !bad) {
        float all = 0.0f;
        int j0 = 0;
        for (; j0 + 16 <= n_experts; j0 += 16) {       // batches of LDS reads, then the ordered adds
            float v[16];
#pragma unroll
            for (int k = 0; k < 16; ++k) v[k] = sh.expv[j0 + k];
#pragma unroll
            for (int k = 0; k < 16; ++k) all = all + v[k];
        }
        for (int j = j0; j < n_experts; ++j) all = all + sh.expv[j];
        if (!(all > 0.0f) || !(all < __builtin_inff())) bad = 1;
        float chosen = 0.0f;
        if (!bad) {
            for (int j = 0; j < topk; ++j) {
                sh.w[j] = sh.expv[sh.sel[j]] / all;
                chosen = chosen + sh.w[j];
            }
            if (!(chosen > 0.0f) || !(chosen < __builtin_inff())) bad = 1;
        }
        if (!bad)
            for (int j = 0; j < topk; ++j) {
                const float share = sh.w[j] / chosen;
                sh.w[j] = share * per_expert_scale[sh.sel[j]];
            }
        sh.bad = bad;
    }
    __syncthreads();
    bad = sh.bad;
    if (e < topk) {
        int place = e;
        if (bad) {
            sh.out_sel[e] = e;                   // a valid placeholder so that dependent work stays in bounds
            sh.out_w[e] = 0.0f;
        } else {
            const int expert = sh.sel[e];
            if (sorted_by_id) {
                place = 0;
                for (int j = 0; j < topk; ++j) place += sh.sel[j] < expert;
            }
            sh.out_sel[place] = expert;
            sh.out_w[place] = want_weights ? sh.w[e] : 0.0f;
        }
    }
    __syncthreads();
}

// The same selection for one wave on its own, without LDS or barriers: which expert stands at position `place` of
// the chosen experts in ascending-id order (the order in which the reference's callers run them,
// gemma4_text.c:7923-7930).  Returns -1 when a logit or a per-expert scale is not finite (the reference rejects the
// call).  n_experts <= 256, every lane of the wave active.
//
// "Rank below topk" is a selection of the topk largest logits with ties going to the smaller index.  The wave finds
// the topk-th largest value by a radix search over order-preserving integer keys (a compare and a population count
// per bit, from the top; the search ends as soon as exactly topk keys reach the candidate, which for distinct logits
// happens after the few bits in which the topk-th and the next value differ), takes everything above it and the
// lowest-indexed of the values equal to it.  Q = registers of keys per lane = ceil(n_experts / 64).
constexpr int ROUTER_WAVE_MAX_EXPERTS = 256;

template <int Q>
__device__ __forceinline__ int router_select_wave_keys(const float *__restrict__ logits,
                                                       const float *__restrict__ per_expert_scale, int n_experts, int topk,
                                                       int place, int second_place, int &second_expert) {
    const int lane = threadIdx.x & 63;
    uint32_t key[Q];
    bool finite = true;
#pragma unroll
    for (int q = 0; q < Q; ++q) {
        const int e = q * 64 + lane;
        key[q] = 0u;                                                     // below every real key
        if (e < n_experts) {
            const float v = logits[e] + 0.0f;                            // -0 becomes +0: they compare equal
            const float sc = per_expert_scale[e];
            finite = finite && (__builtin_fabsf(v) < __builtin_inff()) && (__builtin_fabsf(sc) < __builtin_inff());
            const uint32_t bits = __float_as_uint(v);
            key[q] = (bits & 0x80000000u) ? ~bits : (bits | 0x80000000u);
        }
    }
    if (__ballot(!finite) != 0ull) return -1;
    // the largest threshold that at least topk keys reach
    uint32_t threshold = 0u;
    for (int bit = 31; bit >= 0; --bit) {
        const uint32_t candidate = threshold | (1u << bit);
        int reach = 0;
#pragma unroll
        for (int q = 0; q < Q; ++q) reach += __popcll(__ballot(key[q] >= candidate));
        if (reach >= topk) threshold = candidate;
        if (reach == topk) break;                                        // these topk keys are the selection
    }
    int above = 0;
#pragma unroll
    for (int q = 0; q < Q; ++q) above += __popcll(__ballot(key[q] > threshold));
    const int ties_wanted = topk - above;                                // of the keys equal to the threshold
    const uint64_t below_me = (1ull << lane) - 1ull;
    bool chosen[Q];
    int ties_before = 0;
#pragma unroll
    for (int q = 0; q < Q; ++q) {
        const uint64_t equal = __ballot(key[q] == threshold);
        const int my_tie = ties_before + __popcll(equal & below_me);
        chosen[q] = key[q] > threshold || (key[q] == threshold && my_tie < ties_wanted);
        ties_before += __popcll(equal);
    }
    // position of every chosen expert in ascending-id order; the ones at `place` and `second_place` answer
    int expert = -1, before = 0;
    second_expert = -1;
#pragma unroll
    for (int q = 0; q < Q; ++q) {
        const uint64_t mask = __ballot(chosen[q]);
        const int position = before + __popcll(mask & below_me);
        const uint64_t hit = __ballot(chosen[q] && position == place);
        if (hit != 0ull) expert = q * 64 + (int)__builtin_ctzll(hit);
        const uint64_t second_hit = __ballot(chosen[q] && position == second_place);
        if (second_hit != 0ull) second_expert = q * 64 + (int)__builtin_ctzll(second_hit);
        before += __popcll(mask);
    }
    return expert;
}

// Experts at two positions of the selection at once (second_place < 0: none asked for).
__device__ __forceinline__ int router_select_wave_pair(const float *__restrict__ logits,
                                                       const float *__restrict__ per_expert_scale, int n_experts, int topk,
                                                       int place, int second_place, int &second_expert) {
    if (n_experts <= 64)
        return router_select_wave_keys<1>(logits, per_expert_scale, n_experts, topk, place, second_place, second_expert);
    if (n_experts <= 128)
        return router_select_wave_keys<2>(logits, per_expert_scale, n_experts, topk, place, second_place, second_expert);
    return router_select_wave_keys<4>(logits, per_expert_scale, n_experts, topk, place, second_place, second_expert);
}

__device__ __forceinline__ int router_select_wave(const float *__restrict__ logits,
                                                  const float *__restrict__ per_expert_scale, int n_experts, int topk,
                                                  int place) {
    int unused;
    return router_select_wave_pair(logits, per_expert_scale, n_experts, topk, place, -1, unused);
}

}  // namespace mi355
