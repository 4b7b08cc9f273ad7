// Format-level device entries: the two dequantisers that define the weight formats and the fixture router.  None of
// them is on a hot path (the matvec kernels decode in registers); they exist so that the formats themselves, not
// only the matvecs built on them, have a device statement that is checked bit for bit.
//
//   q4_decode            reference salt_q4_decode (src/kernels.c:188-208): out[k] = fl(fl((float)q * s) + b) with the
//                        scale and bias of group k / 64; any byte alignment; biases may be null.
//   nvfp4_dequant        reference salt_nvfp4_dequantize_weights_reference (src/nvfp4.c:132-155):
//                        out = fl(e2m1(code) * fl(e4m3(scale) * (1 / stored divisor))).
//   router_fixture       reference salt_router (src/router.c:22-57): scores are hashes of (state, layer, expert) in
//                        double arithmetic, selection by repeated strict maximum of the biased score (the smaller
//                        index wins ties), weights are the unbiased scores.
#include "mi355_internal.h"

namespace mi355 {
namespace {

typedef const uint8_t __attribute__((address_space(1))) *global_u8_ptr;

__device__ __forceinline__ uint32_t load_u16(global_u8_ptr p) { return (uint32_t)p[0] | ((uint32_t)p[1] << 8); }

__global__ __launch_bounds__(256) void q4_decode_kernel(const uint8_t *vals_, const uint8_t *scales_, const uint8_t *biases_,
                                                        size_t n, float *out) {
    const size_t k = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (k >= n) return;
    const global_u8_ptr vals = (global_u8_ptr)(uintptr_t)vals_, scales = (global_u8_ptr)(uintptr_t)scales_;
    const global_u8_ptr biases = (global_u8_ptr)(uintptr_t)biases_;
    const uint32_t byte = vals[k >> 1];
    const uint32_t q = (k & 1) ? byte >> 4 : byte & 15u;
    const size_t g = k >> 6;
    const float s = __uint_as_float(load_u16(scales + 2 * g) << 16);
    const float b = biases ? __uint_as_float(load_u16(biases + 2 * g) << 16) : 0.0f;
    const float product = (float)q * s;
    out[k] = product + b;
}

__device__ __forceinline__ float e2m1_value(uint32_t code) {
    const uint32_t m = code & 7u;
    const float mag = m == 0 ? 0.0f : m == 1 ? 0.5f : (1.0f + 0.5f * (float)(m & 1u)) * (float)(1u << ((m >> 1) - 1u));
    return (code & 8u) && m != 0 ? -mag : mag;           // the reference's table holds +0 for code 8
}

__global__ __launch_bounds__(256) void nvfp4_dequant_kernel(const uint8_t *packed, const uint8_t *scales,
                                                            float weight_global_scale, int C, size_t n, float *out) {
    const size_t index = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (index >= n) return;
    const uint32_t byte = packed[index >> 1];
    const uint32_t code = (index & 1) ? byte >> 4 : byte & 15u;
    const size_t row = index / (size_t)C, col = index - row * (size_t)C;
    const float scale = __builtin_amdgcn_cvt_f32_fp8((int)scales[row * (size_t)(C / 16) + col / 16], 0);
    const float scaled = scale * weight_global_scale;
    out[index] = e2m1_value(code) * scaled;
}

__device__ __forceinline__ uint64_t mix64(uint64_t x) {                  // splitmix64 finaliser (router.c:11-16)
    x += 0x9E3779B97F4A7C15ull;
    x = (x ^ (x >> 30)) * 0xBF58476D1CE4E5B9ull;
    x = (x ^ (x >> 27)) * 0x94D049BB133111EBull;
    return x ^ (x >> 31);
}
__device__ __forceinline__ uint64_t hash3(uint64_t a, uint64_t b, uint64_t c) {
    return mix64(a ^ mix64(b * 0x100000001B3ull + c));
}

constexpr int FIXTURE_MAX_EXPERTS = 1024;

// One workgroup, one thread per expert.  The position of an expert in the reference's selection list is its rank:
// the number of experts with a larger selection score plus the number of equal ones with a smaller index.
__global__ __launch_bounds__(FIXTURE_MAX_EXPERTS) void router_fixture_kernel(int n_experts, int topk, uint64_t state, int layer,
                                                                             double locality, int *idx, float *w) {
    __shared__ float choose[FIXTURE_MAX_EXPERTS];
    const int e = threadIdx.x;
    float score = 0.0f, mine = 0.0f;
    if (e < n_experts) {
        const double acc = (double)(hash3(state, (uint64_t)layer, (uint64_t)e) & 0xFFFFFFull) / (double)0x1000000;
        const double bias = (double)(hash3(state ^ 0xB1A5ull, (uint64_t)layer, (uint64_t)e) & 0xFFFFFFull) / (double)0x1000000;
        const double centred = bias - 0.5;
        const double nudge = centred * 0.1;
        double sel = acc + nudge;
        if (locality > 0.0) {
            const double pop = 1.0 / (1.0 + (double)(e % 64));
            const double lift = locality * pop;
            const double factor = 1.0 + lift;
            sel = acc * factor;
        }
        score = (float)acc;
        mine = (float)sel;
        choose[e] = mine;
    }
    __syncthreads();
    if (e < n_experts) {
        int rank = 0;
        for (int j = 0; j < n_experts; ++j) {
            const float other = choose[j];
            rank += (other > mine) || (other == mine && j < e);
        }
        if (rank < topk) { idx[rank] = e; w[rank] = score; }
    }
}

}  // namespace

int q4_decode_launch(const uint8_t *vals, const uint8_t *scales, const uint8_t *biases, size_t n, float *out,
                     hipStream_t stream) {
    if (n == 0) return 0;
    if ((n + 255) / 256 > 0x7fffffffull) return -1;
    hipLaunchKernelGGL(q4_decode_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, stream, vals, scales, biases, n, out);
    return hipGetLastError() == hipSuccess ? 0 : -1;
}

int nvfp4_dequant_launch(const uint8_t *packed, const uint8_t *scales, float weight_global_scale, int R, int C, float *out,
                         hipStream_t stream) {
    const size_t n = (size_t)R * (size_t)C;
    if ((n + 255) / 256 > 0x7fffffffull) return -1;
    hipLaunchKernelGGL(nvfp4_dequant_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, stream, packed, scales,
                       weight_global_scale, C, n, out);
    return hipGetLastError() == hipSuccess ? 0 : -1;
}

int router_fixture_launch(int n_experts, int topk, uint64_t state, int layer, double locality, int *idx, float *w,
                          hipStream_t stream) {
    if (n_experts < 1 || n_experts > FIXTURE_MAX_EXPERTS || topk < 1 || topk > n_experts) return -1;
    const int threads = (n_experts + 63) & ~63;
    hipLaunchKernelGGL(router_fixture_kernel, dim3(1), dim3(threads), 0, stream, n_experts, topk, state, layer, locality, idx, w);
    return hipGetLastError() == hipSuccess ? 0 : -1;
}

}  // namespace mi355
