// Prefill-sized affine-Q4 matmul on the MFMA units (tolerance class).
//
// When many tokens meet one weight matrix the work is a dense contraction and
// the 32-chain order of the decode kernels cannot be kept at matrix-core speed.
// This kernel computes Y[token][row] = sum_c (q*s + b)[row][c] * x[token][c]
// with fp32-level accuracy but in a different summation order; callers opt in
// and are told so (the engine's bit-exact path remains the tiled kernels).
//
// How the affine weights reach the matrix cores without losing bits:
//  * per 64-column scale group,  sum_c (q s + b) x = s * sum_c q x + b * sum_c x.
//    The integer codes are exact in bf16, so only sum_c q x goes through MFMA;
//    scale and bias are applied per group in fp32 on the VALU.
//  * a nibble becomes the bf16 value 16 + q with three bit operations
//    (0x4180 | q << 3); the surplus 16 * sum_c x is removed with the bias term.
//  * the fp32 activation is split once into three bf16 planes
//    (x = hi + mid + lo to 2^-24), each of which is an exact MFMA operand;
//    accumulation is fp32.
//
// Tiling: a workgroup of four waves computes 64 tokens x 64 weight rows, each
// wave a 32 x 32 block with v_mfma_f32_32x32x16_bf16 (tokens are the M rows,
// weight rows the N columns, so a lane owns one weight row and needs one
// (scale, bias) pair per group).  Per group the planes, the packed codes, the
// (scale, bias - 16*scale) pairs and the group sums of x are staged in LDS with
// the next group's loads in flight.
#include "device_math.h"
#include "mi355_internal.h"

#include <stddef.h>

namespace mi355 {
namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef const uint64_t __attribute__((address_space(4))) *uniform_u64_ptr;
typedef const u32x4 __attribute__((address_space(1))) *global_u128_ptr;
typedef const uint16_t __attribute__((address_space(1))) *global_u16_ptr;
typedef const float __attribute__((address_space(1))) *global_f32_ptr;

constexpr int TM = 64, TN = 64;            // tokens x weight rows per workgroup
constexpr int X_PITCH = 144;               // bytes per staged token row of one plane: 64 bf16 + 16 pad
constexpr int W_PITCH = 36;                // bytes per staged weight row of one group: 32 + 4 pad

static_assert(sizeof(MfmaJob) == 64, "find_job reads a job record as eight 64-bit words");

__device__ __forceinline__ MfmaJob find_job(const MfmaLaunch &L, int tile) {
    if (L.table == nullptr) return L.one;
    const uniform_u64_ptr words = (uniform_u64_ptr)(uintptr_t)L.table;
    const int njobs = L.njobs_dev ? *(const int __attribute__((address_space(4))) *)(uintptr_t)L.njobs_dev : L.njobs;
    int lo = 0, hi = njobs - 1;
    while (lo < hi) {
        const int mid = (lo + hi + 1) >> 1;
        if ((int)(uint32_t)words[8 * mid + 7] <= tile) lo = mid; else hi = mid - 1;
    }
    const uniform_u64_ptr rec = words + 8 * lo;
    MfmaJob job;
    job.vals = (const uint8_t *)rec[0];
    job.scales = (const uint8_t *)rec[1];
    job.biases = (const uint8_t *)rec[2];
    job.planes = (const uint16_t *)rec[3];
    job.xsum = (const float *)rec[4];
    job.y = (float *)rec[5];
    job.tokens = (int)(uint32_t)rec[6];
    job.rows = (int)(rec[6] >> 32);
    job.tile0 = (int)(uint32_t)rec[7];
    job.reserved = 0;
    return job;
}

__device__ __forceinline__ float bf16_to_f32(uint32_t half) { return __uint_as_float(half << 16); }

// Eight nibbles -> eight bf16 values 16 + q, in column order.
__device__ __forceinline__ bf16x8 codes_to_bf16(uint32_t w) {
    const uint32_t even = (w << 3) & 0x78787878u;        // q0, q2, q4, q6 (each << 3) in bytes 0..3
    const uint32_t odd = (w >> 1) & 0x78787878u;         // q1, q3, q5, q7
    u32x4 r;
    r.x = __builtin_amdgcn_perm(odd, even, 0x0C040C00u) | 0x41804180u;
    r.y = __builtin_amdgcn_perm(odd, even, 0x0C050C01u) | 0x41804180u;
    r.z = __builtin_amdgcn_perm(odd, even, 0x0C060C02u) | 0x41804180u;
    r.w = __builtin_amdgcn_perm(odd, even, 0x0C070C03u) | 0x41804180u;
    return __builtin_bit_cast(bf16x8, r);
}

__global__ __launch_bounds__(256) void q4_mfma_kernel(const MfmaLaunch L) {
    __shared__ __attribute__((aligned(16))) uint8_t xs[3 * TM * X_PITCH];
    __shared__ __attribute__((aligned(16))) uint8_t ws[TN * W_PITCH];
    __shared__ float2 ms[TN];
    __shared__ float xg[TM];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave >> 1, wn = wave & 1;
    const int l32 = lane & 31, half = lane >> 5;

    if (L.total_tiles_dev &&
        (int)blockIdx.x >= *(const int __attribute__((address_space(4))) *)(uintptr_t)L.total_tiles_dev)
        return;                                     // uniform: the whole workgroup leaves
    const MfmaJob job = find_job(L, blockIdx.x);
    const int C = L.cols, ngrp = C >> 6;
    const int ntiles = (job.rows + TN - 1) / TN;
    const int t = blockIdx.x - job.tile0;
    const int tok0 = (t / ntiles) * TM, row0 = (t % ntiles) * TN;
    const int toks_here = job.tokens - tok0 < TM ? job.tokens - tok0 : TM;
    const int rows_here = job.rows - row0 < TN ? job.rows - row0 : TN;

    // staging geometry of this thread
    // planes: 3 * 64 tokens * 8 segments of 16 bytes = 1536 pieces, 6 per thread
    const global_u16_ptr planes = (global_u16_ptr)(uintptr_t)job.planes;
    uint32_t x_src[6], x_dst[6];
#pragma unroll
    for (int i = 0; i < 6; ++i) {
        const int p = tid + i * 256;
        const int plane = p >> 9, tok = (p >> 3) & 63, seg = p & 7;
        const int tc = tok < toks_here ? tok : toks_here - 1;
        x_src[i] = (uint32_t)(tok0 + tc) * (uint32_t)C + seg * 8;          // element offset inside the plane
        x_dst[i] = plane * (TM * X_PITCH) + tok * X_PITCH + seg * 16;
    }
    const size_t plane_stride = L.plane_stride;
    // codes: 64 rows * 2 pieces of 16 bytes, threads 0..127
    const int w_row = (tid >> 1) & 63, w_half = tid & 1;
    const int w_rc = w_row < rows_here ? w_row : rows_here - 1;
    const global_u128_ptr w_src = (global_u128_ptr)((uintptr_t)job.vals + (size_t)(row0 + w_rc) * (C >> 1) + w_half * 16);
    // (scale, bias): threads 128..191; group sums of x: threads 192..255
    const int m_row = tid & 63;
    const int m_rc = m_row < rows_here ? m_row : rows_here - 1;
    const int g_tc = m_row < toks_here ? m_row : toks_here - 1;
    const global_u16_ptr scales = (global_u16_ptr)(uintptr_t)job.scales + (size_t)(row0 + m_rc) * ngrp;
    const global_u16_ptr biases = job.biases ? (global_u16_ptr)(uintptr_t)job.biases + (size_t)(row0 + m_rc) * ngrp
                                             : (global_u16_ptr)0;
    const global_f32_ptr xsum = (global_f32_ptr)(uintptr_t)job.xsum + (size_t)(tok0 + g_tc) * ngrp;

    u32x4 xreg[6], wreg;
    uint32_t sreg = 0, breg = 0;
    float greg = 0.0f;
    auto issue = [&](int g) {
#pragma unroll
        for (int i = 0; i < 6; ++i) {
            const int plane = (tid + i * 256) >> 9;
            xreg[i] = *(global_u128_ptr)(planes + (size_t)plane * plane_stride + x_src[i] + (uint32_t)g * 64u);
        }
        if (tid < 128) wreg = w_src[g * 2];
        else if (tid < 192) { sreg = scales[g]; breg = biases ? (uint32_t)biases[g] : 0u; }
        else greg = xsum[g];
    };
    auto commit = [&]() {
#pragma unroll
        for (int i = 0; i < 6; ++i) *reinterpret_cast<u32x4 *>(xs + x_dst[i]) = xreg[i];
        if (tid < 128) {
            uint32_t *dst = reinterpret_cast<uint32_t *>(ws + w_row * W_PITCH + w_half * 16);
            dst[0] = wreg.x; dst[1] = wreg.y; dst[2] = wreg.z; dst[3] = wreg.w;
        } else if (tid < 192) {
            const float s = bf16_to_f32(sreg), b = bf16_to_f32(breg);
            ms[m_row] = make_float2(s, b - 16.0f * s);
        } else {
            xg[m_row] = greg;
        }
    };

    f32x16 acc;
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[i] = 0.0f;

    issue(0);
    for (int g = 0; g < ngrp; ++g) {
        commit();
        __syncthreads();
        if (g + 1 < ngrp) issue(g + 1);

        f32x16 part;
#pragma unroll
        for (int i = 0; i < 16; ++i) part[i] = 0.0f;
        const uint8_t *wrow = ws + (wn * 32 + l32) * W_PITCH + half * 4;
        const uint8_t *xrow = xs + (wm * 32 + l32) * X_PITCH + half * 16;
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) {
            const bf16x8 b = codes_to_bf16(*reinterpret_cast<const uint32_t *>(wrow + ks * 8));
#pragma unroll
            for (int plane = 0; plane < 3; ++plane) {
                const u32x4 raw = *reinterpret_cast<const u32x4 *>(xrow + plane * (TM * X_PITCH) + ks * 32);
                part = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, raw), b, part, 0, 0, 0);
            }
        }
        const float2 sc = ms[wn * 32 + l32];
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const int tok = (i >> 2) * 8 + half * 4 + (i & 3);
            acc[i] = __builtin_fmaf(sc.x, part[i], acc[i]);
            acc[i] = __builtin_fmaf(sc.y, xg[wm * 32 + tok], acc[i]);
        }
        __syncthreads();
    }

    const int row = wn * 32 + l32;
    if (row < rows_here) {
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const int tok = wm * 32 + (i >> 2) * 8 + half * 4 + (i & 3);
            if (tok < toks_here) job.y[(size_t)(tok0 + tok) * job.rows + row0 + row] = acc[i];
        }
    }
}

// fp32 rows -> three bf16 planes and per-64-column sums.  Row r of the output
// is row row_map[r] of the input when a map is given (the grouped MoE gather).
__device__ __forceinline__ uint32_t f32_to_bf16_rne(float v) {
    const uint32_t bits = __float_as_uint(v);
    return (bits + 0x7FFFu + ((bits >> 16) & 1u)) >> 16;
}

// With GATED the value split is gelu_tanh(gate) * x (the expert activation,
// reference gemma4_text.c:8749-9137 "down input"), so the activations never
// make a round trip through memory in fp32.
template <bool GATED>
__global__ __launch_bounds__(256) void x_split_kernel(const float *__restrict__ x, const float *__restrict__ gate,
                                                      const int *__restrict__ row_map, int map_divisor, int x_stride,
                                                      int rows, int cols, uint16_t *__restrict__ planes,
                                                      size_t plane_stride, float *__restrict__ xsum) {
    const int row = blockIdx.x;
    const int c0 = (blockIdx.y * 256 + threadIdx.x) * 8;
    const bool live = c0 < cols;
    float v[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    if (live) {
        const int src_row = row_map ? row_map[row] / map_divisor : row;
        const float4 *src = reinterpret_cast<const float4 *>(x + (size_t)src_row * x_stride + c0);
        const float4 a = src[0], b = src[1];
        v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w; v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
        if (GATED) {
            const float4 *gsrc = reinterpret_cast<const float4 *>(gate + (size_t)src_row * x_stride + c0);
            const float4 ga = gsrc[0], gb = gsrc[1];
            const float gv[8] = {ga.x, ga.y, ga.z, ga.w, gb.x, gb.y, gb.z, gb.w};
#pragma unroll
            for (int j = 0; j < 8; ++j) v[j] = det_gelu_tanh(gv[j]) * v[j];
        }
    }
    uint32_t hi[4], mid[4], lo[4];
    float sum = 0.0f;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        const uint32_t h = f32_to_bf16_rne(v[j]);
        const float r1 = v[j] - bf16_to_f32(h);
        const uint32_t m = f32_to_bf16_rne(r1);
        const float r2 = r1 - bf16_to_f32(m);
        const uint32_t l = f32_to_bf16_rne(r2);
        if (j & 1) { hi[j >> 1] |= h << 16; mid[j >> 1] |= m << 16; lo[j >> 1] |= l << 16; }
        else { hi[j >> 1] = h; mid[j >> 1] = m; lo[j >> 1] = l; }
        sum += v[j];
    }
    // eight lanes cover one 64-column group
    sum += __shfl_xor(sum, 1, 64);
    sum += __shfl_xor(sum, 2, 64);
    sum += __shfl_xor(sum, 4, 64);
    if (live) {
        uint16_t *dst = planes + (size_t)row * cols + c0;
        *reinterpret_cast<uint4 *>(dst) = make_uint4(hi[0], hi[1], hi[2], hi[3]);
        *reinterpret_cast<uint4 *>(dst + plane_stride) = make_uint4(mid[0], mid[1], mid[2], mid[3]);
        *reinterpret_cast<uint4 *>(dst + 2 * plane_stride) = make_uint4(lo[0], lo[1], lo[2], lo[3]);
        if ((threadIdx.x & 7) == 0) xsum[(size_t)row * (cols >> 6) + (c0 >> 6)] = sum;
    }
}

}  // namespace

int q4_mfma_launch(const MfmaLaunch &L, hipStream_t stream) {
    if (L.total_tiles < 1 || L.cols < 64 || (L.cols & 63)) return -1;
    hipLaunchKernelGGL(q4_mfma_kernel, dim3(L.total_tiles), dim3(256), 0, stream, L);
    return hipGetLastError() == hipSuccess ? 0 : -1;
}

int x_split_launch(const float *x, const float *gate, const int *row_map, int map_divisor, int x_stride, int rows,
                   int cols, uint16_t *planes, size_t plane_stride, float *xsum, hipStream_t stream) {
    if (rows < 1 || cols < 64 || (cols & 63)) return -1;
    const dim3 grid(rows, (cols / 8 + 255) / 256);
    if (gate)
        hipLaunchKernelGGL(x_split_kernel<true>, grid, dim3(256), 0, stream, x, gate, row_map, map_divisor, x_stride,
                           rows, cols, planes, plane_stride, xsum);
    else
        hipLaunchKernelGGL(x_split_kernel<false>, grid, dim3(256), 0, stream, x, gate, row_map, map_divisor, x_stride,
                           rows, cols, planes, plane_stride, xsum);
    return hipGetLastError() == hipSuccess ? 0 : -1;
}

int mfma_tiles(int tokens, int rows) { return ((tokens + TM - 1) / TM) * ((rows + TN - 1) / TN); }

}  // namespace mi355
