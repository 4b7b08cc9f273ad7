// 8-bit affine matrix times fp32 vector in the reference's order (router gates and the shared-expert gate,
// reference src/kernels.c:343-370): one accumulator per row walks the columns left to right,
//     acc = acc + ((float)byte * scale + bias) * x[c]
// with every operation rounded separately and the scale and bias of the 64-element group that holds the flat element
// row * cols + c.  The chain of one row cannot be split, and a dependent fp32 addition issues only every dozen clocks
// from a lone wave, so the chain itself bounds the time (about 15 us for 2816 columns); the kernels differ in what
// else sits on the adding wave.
#include "mi355_internal.h"

namespace mi355 {
namespace {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef const u32x4 __attribute__((address_space(1))) *global_u128_ptr;
typedef const uint16_t __attribute__((address_space(1))) *global_u16_ptr;
typedef const float __attribute__((address_space(4))) *uniform_f32_ptr;

__device__ __forceinline__ float bf16_bits(uint32_t half) { return __uint_as_float(half << 16); }

// More than 4096 columns (cols % 64 == 0, 16-byte aligned values): a lane owns a row and does all of its work;
// activations reach it as scalar operands.  blockIdx.y is the activation row.
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

// Up to 4096 columns.  A workgroup owns 8 rows and one activation row.  The chain of a row is one addition per column
// and nothing else can be taken off it, so the work is split by kind: three waves turn bytes into rounded products
// ((float)byte * scale + bias) * x and leave them in LDS, and the fourth wave only adds them, in column order, one
// lane per row, reading the next 32 products while it adds the current 32.  Products travel in chunks of 704 columns
// through two LDS buffers (few chunks, so few barriers); all bytes of the 8 rows are held in registers from the
// start, so the memory latency is paid once.
constexpr int CH_ROWS = 8;
constexpr int CH_COLS = 704;                       // 44 segments of 16 bytes per row
constexpr int CH_SEGS = CH_COLS / 16;
constexpr int CH_ITEMS = CH_ROWS * CH_SEGS;        // 352 (row, segment) items per chunk over 192 producer lanes
constexpr int CH_PER_LANE = (CH_ITEMS + 191) / 192;
constexpr int CH_PITCH = CH_COLS + 4;              // floats; the eight adding lanes then touch distinct banks
constexpr int CH_MAX_COLS = 4096;
constexpr int CH_MAX_CHUNKS = (CH_MAX_COLS + CH_COLS - 1) / CH_COLS;

__global__ __launch_bounds__(256) void q8_chain_kernel(Q8Launch L) {
    __shared__ float x_lds[CH_MAX_COLS];
    __shared__ uint16_t scale_lds[CH_ROWS][CH_MAX_COLS / 64], bias_lds[CH_ROWS][CH_MAX_COLS / 64];     // bf16 bits
    // the adder reads up to 64 floats past the end of a chunk (and discards them): hence the tail
    __shared__ __attribute__((aligned(16))) float ring[2 * CH_ROWS * CH_PITCH + 64];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int row0 = blockIdx.x * CH_ROWS;
    const int rows_here = L.rows - row0 < CH_ROWS ? L.rows - row0 : CH_ROWS;
    const int C = L.cols, groups = C / 64;
    const int nchunk = (C + CH_COLS - 1) / CH_COLS;
    const float *x = L.x + (size_t)blockIdx.y * L.x_stride;

    // producer items: item = row * 44 + segment.  All of a lane's bytes are requested before anything else happens,
    // unconditionally (a column past the row re-reads the row's last segment), so the loads are straight-line code
    // and each use waits only for its own load.
    const int pid = tid >= 64 ? tid - 64 : 0;
    int prow[CH_PER_LANE], pseg[CH_PER_LANE];
    u32x4 bytes[CH_MAX_CHUNKS][CH_PER_LANE];
#pragma unroll
    for (int j = 0; j < CH_PER_LANE; ++j) {
        const int item = pid + 192 * j < CH_ITEMS ? pid + 192 * j : CH_ITEMS - 1;
        prow[j] = item / CH_SEGS;
        pseg[j] = item % CH_SEGS;
    }
#pragma unroll
    for (int k = 0; k < CH_MAX_CHUNKS; ++k)
#pragma unroll
        for (int j = 0; j < CH_PER_LANE; ++j) {
            const int row = prow[j] < rows_here ? prow[j] : rows_here - 1;
            const int col = k * CH_COLS + pseg[j] * 16;
            bytes[k][j] = *(global_u128_ptr)(uintptr_t)(L.vals + (size_t)(row0 + row) * C + (col < C ? col : C - 16));
        }
    for (int c = tid; c < C; c += 256) x_lds[c] = x[c];
    for (int i = tid; i < CH_ROWS * groups; i += 256) {
        const int r = i / groups, g = i % groups;
        const size_t at = (size_t)(row0 + (r < rows_here ? r : rows_here - 1)) * groups + g;
        scale_lds[r][g] = ((const uint16_t *)L.scales)[at];
        bias_lds[r][g] = L.biases ? ((const uint16_t *)L.biases)[at] : (uint16_t)0;
    }
    __syncthreads();

    float acc = 0.0f;
    const int crow = lane < CH_ROWS ? lane : 0;
    // step i: producers fill ring[i % 2] with chunk i while the adder walks chunk i - 1 in ring[(i - 1) % 2]
#pragma unroll
    for (int i = 0; i <= CH_MAX_CHUNKS; ++i) {
        if (i > nchunk) continue;                 // uniform over the workgroup
        if (wave != 0) {
#pragma unroll
            for (int j = 0; j < CH_PER_LANE; ++j) {
                const int col = i * CH_COLS + pseg[j] * 16;
                if (i < CH_MAX_CHUNKS && pid + 192 * j < CH_ITEMS && col < C) {
                    const u32x4 v = bytes[i < CH_MAX_CHUNKS ? i : 0][j];
                    const uint32_t word[4] = {v.x, v.y, v.z, v.w};
                    const float s = bf16_bits(scale_lds[prow[j]][col / 64]), b = bf16_bits(bias_lds[prow[j]][col / 64]);
                    float *out = &ring[((i & 1) * CH_ROWS + prow[j]) * CH_PITCH + pseg[j] * 16];
#pragma unroll
                    for (int p = 0; p < 4; ++p) {
                        const float4 xv = *(const float4 *)&x_lds[col + 4 * p];
                        const float xs[4] = {xv.x, xv.y, xv.z, xv.w};
                        float prod[4];
#pragma unroll
                        for (int q = 0; q < 4; ++q) {
                            float value = (float)((word[p] >> (8 * q)) & 0xffu) * s;
                            value = value + b;
                            prod[q] = value * xs[q];
                        }
                        *(float4 *)&out[4 * p] = make_float4(prod[0], prod[1], prod[2], prod[3]);
                    }
                }
            }
        } else if (i >= 1 && lane < CH_ROWS) {
            const int c0 = (i - 1) * CH_COLS;
            const int count = C - c0 < CH_COLS ? C - c0 : CH_COLS;          // a multiple of 64
            const float *in = &ring[(((i - 1) & 1) * CH_ROWS + crow) * CH_PITCH];
            float4 a[8], b[8];
            auto fetch = [&](float4 (&dst)[8], int at) {
#pragma unroll
                for (int k = 0; k < 8; ++k) dst[k] = *(const float4 *)&in[at + 4 * k];
            };
            auto add = [&](const float4 (&src)[8]) {
#pragma unroll
                for (int k = 0; k < 8; ++k) {
                    acc = acc + src[k].x;
                    acc = acc + src[k].y;
                    acc = acc + src[k].z;
                    acc = acc + src[k].w;
                }
            };
            fetch(a, 0);
            for (int at = 0; at < count; at += 64) {        // the last fetch of a reads past the chunk and is dropped
                fetch(b, at + 32);
                add(a);
                fetch(a, at + 64);
                add(b);
            }
        }
        __syncthreads();
    }
    if (wave == 0 && lane < rows_here) L.y[(size_t)blockIdx.y * L.y_stride + row0 + lane] = acc;
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
    if (fast && L.cols <= CH_MAX_COLS)
        q8_chain_kernel<<<dim3((L.rows + CH_ROWS - 1) / CH_ROWS, L.tokens), dim3(256), 0, stream>>>(L);
    else if (fast) q8_rows_kernel<<<grid, dim3(64), 0, stream>>>(L);
    else q8_generic_kernel<<<grid, dim3(64), 0, stream>>>(L);
    return hipGetLastError() == hipSuccess ? 0 : -1;
}

}  // namespace mi355
