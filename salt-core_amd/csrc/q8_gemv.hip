// 8-bit affine matrix times fp32 vector in the reference's order (router gates and the shared-expert gate,
// reference src/kernels.c:343-370): one accumulator per row walks the columns left to right,
//     acc = acc + ((float)byte * scale + bias) * x[c]
// with every operation rounded separately and the scale and bias of the 64-element group that holds the flat element
// row * cols + c.  The chain of one row cannot be split, so a lane owns a row; lanes of a wave own 64 consecutive
// rows and the activations reach them as scalar operands.
#include "mi355_internal.h"

namespace mi355 {
namespace {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef const u32x4 __attribute__((address_space(1))) *global_u128_ptr;
typedef const uint16_t __attribute__((address_space(1))) *global_u16_ptr;
typedef const float __attribute__((address_space(4))) *uniform_f32_ptr;

__device__ __forceinline__ float bf16_bits(uint32_t half) { return __uint_as_float(half << 16); }

// cols % 64 == 0 and 16-byte aligned values: groups never straddle rows.  blockIdx.y is the activation row.
__global__ __launch_bounds__(64) void q8_rows_kernel(Q8Launch L) {
    const int lane = threadIdx.x;
    const int row0 = blockIdx.x * 64;
    const int rows_here = L.rows - row0 < 64 ? L.rows - row0 : 64;
    const int row = row0 + (lane < rows_here ? lane : rows_here - 1);
    const int token = blockIdx.y;
    const int groups = L.cols / 64;
    const global_u128_ptr w = (global_u128_ptr)(uintptr_t)(L.vals + (size_t)row * L.cols);
    const global_u16_ptr sc = (global_u16_ptr)(uintptr_t)L.scales + (size_t)row * groups;
    const global_u16_ptr bi = (global_u16_ptr)(uintptr_t)L.biases + (size_t)row * groups;
    const uniform_f32_ptr x = (uniform_f32_ptr)(uintptr_t)(L.x + (size_t)token * L.x_stride);
    const bool has_bias = L.biases != nullptr;
    float acc = 0.0f;
    for (int g = 0; g < groups; ++g) {
        const float s = bf16_bits(sc[g]);
        const float b = has_bias ? bf16_bits(bi[g]) : 0.0f;
        u32x4 v[4];
#pragma unroll
        for (int q = 0; q < 4; ++q) v[q] = w[g * 4 + q];
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const uint32_t word[4] = {v[q].x, v[q].y, v[q].z, v[q].w};
#pragma unroll
            for (int p = 0; p < 4; ++p)
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    float value = (float)((word[p] >> (8 * k)) & 0xffu) * s;
                    value = value + b;
                    acc = acc + value * x[g * 64 + q * 16 + p * 4 + k];
                }
        }
    }
    if (lane < rows_here) L.y[(size_t)token * L.y_stride + row] = acc;
}

// Any column count and alignment.
__global__ __launch_bounds__(64) void q8_generic_kernel(Q8Launch L) {
    const int row = blockIdx.x * 64 + threadIdx.x;
    if (row >= L.rows) return;
    const int token = blockIdx.y;
    const float *x = L.x + (size_t)token * L.x_stride;
    float acc = 0.0f;
    for (int c = 0; c < L.cols; ++c) {
        const size_t k = (size_t)row * L.cols + c;
        const size_t g = k / 64;
        const float s = bf16_bits((uint32_t)L.scales[2 * g] | ((uint32_t)L.scales[2 * g + 1] << 8));
        const float b = L.biases ? bf16_bits((uint32_t)L.biases[2 * g] | ((uint32_t)L.biases[2 * g + 1] << 8)) : 0.0f;
        float value = (float)L.vals[k] * s;
        value = value + b;
        acc = acc + value * x[c];
    }
    L.y[(size_t)token * L.y_stride + row] = acc;
}

}  // namespace

int q8_launch(const Q8Launch &L, hipStream_t stream) {
    if (!L.vals || !L.scales || !L.x || !L.y || L.rows < 1 || L.cols < 1 || L.tokens < 1 || L.tokens > 65535) return -1;
    const dim3 grid((L.rows + 63) / 64, L.tokens);
    const bool fast = L.cols % 64 == 0 && ((uintptr_t)L.vals & 15) == 0 && ((uintptr_t)L.scales & 1) == 0 &&
                      ((uintptr_t)L.biases & 1) == 0 && ((uintptr_t)L.x & 3) == 0;
    if (fast) q8_rows_kernel<<<grid, dim3(64), 0, stream>>>(L);
    else q8_generic_kernel<<<grid, dim3(64), 0, stream>>>(L);
    return hipGetLastError() == hipSuccess ? 0 : -1;
}

}  // namespace mi355
