// Prefill-sized NVFP4 matmul on the MFMA units (tolerance class).
//
// reference src/nvfp4.c:228-256 computes, per output row, sum_c w_c * x_c with
// w_c = e2m1(code) * (e4m3(scale) * weight_global) and x_c the quantised and
// dequantised activation e2m1(code) * (e4m3(scale) / input_global), in its
// 32-chain order.  With hundreds of tokens the work is a dense contraction.
// Both operands factor into a part that is exact in bf16,
//     e2m1(code) * e4m3(block scale)        (two times four significant bits),
// and a per-tensor fp32 factor, so the matrix cores see exact operands, the
// products are exact in fp32 and only the order of the fp32 additions (and the
// two per-tensor factors, applied once at the end) differs from the reference.
//
// Tiling: a workgroup of four waves computes 128 tokens x 128 weight rows, each
// wave 64 x 64 as 2 x 2 blocks of v_mfma_f32_32x32x16_bf16.  Per 64-column chunk
// the activation plane is copied and the weights are decoded (codes through
// v_cvt_scalef32_pk_f32_fp4, scales through v_cvt_f32_fp8, one multiply, the
// upper half kept) into one of two LDS stages with the next chunk's loads in
// flight.  Long contractions with few tiles are split along the columns; the
// partial sums are added in split order by a second kernel.
#include "mi355_internal.h"

#include <stddef.h>

namespace mi355 {
namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef const u32x4 __attribute__((address_space(1))) *global_u128_ptr;
typedef const uint16_t __attribute__((address_space(1))) *global_u16_ptr;

constexpr int TM = 128, TN = 128, KC = 64;
constexpr int PITCH = 144;                     // bytes per staged row: 64 bf16 + 16 pad
constexpr int A_BYTES = TM * PITCH, B_BYTES = TN * PITCH;
constexpr int STAGE_BYTES = A_BYTES + B_BYTES;

struct Geometry {
    int m_tiles, n_tiles, chunks, chunks_per_split;
};

// Whether the activation pass rejected its input: the launch's status word, or the OR of the pass's per-workgroup
// flags (every thread of the workgroup calls this; workgroup 0 then also publishes the outcome).
__device__ __forceinline__ bool rejected(const Fp4MfmaLaunch &L) {
    if (!L.flags) return *(const int __attribute__((address_space(4))) *)(uintptr_t)L.status != 0;
    int bad = 0;
    for (int i = threadIdx.x; i < L.nflags; i += blockDim.x) bad |= L.flags[i];
    const int any_bad = __syncthreads_or(bad);
    if (blockIdx.x == 0 && threadIdx.x == 0) {
        *L.outcome = any_bad ? -1 : 0;
        if (L.outcome_copy) *L.outcome_copy = any_bad ? -1 : 0;
    }
    return any_bad != 0;
}

__device__ __forceinline__ uint32_t pack_upper_halves(float lo, float hi) {
    return __builtin_amdgcn_perm(__float_as_uint(hi), __float_as_uint(lo), 0x07060302u);
}

__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2)))
void fp4_mfma_kernel(const Fp4MfmaLaunch L, const Geometry G) {
    __shared__ __attribute__((aligned(16))) uint8_t stage[2 * STAGE_BYTES];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave >> 1, wn = wave & 1;
    const int l32 = lane & 31, half = lane >> 5;

    // consecutive workgroups share a weight tile
    const int mt = blockIdx.x % G.m_tiles;
    const int nt = (blockIdx.x / G.m_tiles) % G.n_tiles;
    const int split = blockIdx.x / (G.m_tiles * G.n_tiles);
    const int tok0 = mt * TM, row0 = nt * TN;
    const int toks_here = L.tokens - tok0 < TM ? L.tokens - tok0 : TM;
    const int rows_here = L.rows - row0 < TN ? L.rows - row0 : TN;
    const int chunk0 = split * G.chunks_per_split;
    const int chunk1 = chunk0 + G.chunks_per_split < G.chunks ? chunk0 + G.chunks_per_split : G.chunks;
    const int C = L.cols;

    // activation plane: 128 tokens * 8 pieces of 16 bytes, four per thread
    const global_u16_ptr plane = (global_u16_ptr)(uintptr_t)L.plane;
    size_t a_src[4];
    uint32_t a_dst[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int p = tid + i * 256;
        const int tok = p >> 3, seg = p & 7;
        const int tc = tok < toks_here ? tok : toks_here - 1;
        a_src[i] = (size_t)(tok0 + tc) * C + seg * 8;
        a_dst[i] = tok * PITCH + seg * 16;
    }
    // weights: 128 rows * 2 pieces of 32 codes (two scale blocks), one per thread
    const int w_row = tid >> 1, w_half = tid & 1;
    const int w_rc = w_row < rows_here ? w_row : rows_here - 1;
    const global_u128_ptr w_src =
        (global_u128_ptr)((uintptr_t)L.packed + (size_t)(row0 + w_rc) * (C >> 1) + w_half * 16);
    const global_u16_ptr s_src = (global_u16_ptr)((uintptr_t)L.scales + (size_t)(row0 + w_rc) * (C >> 4) + w_half * 2);

    u32x4 areg[4], wreg;
    uint32_t sreg = 0;
    auto issue = [&](int chunk) {
#pragma unroll
        for (int i = 0; i < 4; ++i) areg[i] = *(global_u128_ptr)(plane + a_src[i] + (size_t)chunk * KC);
        wreg = w_src[chunk * 2];
        sreg = s_src[chunk * 2];
    };
    auto commit = [&](uint8_t *base) {
#pragma unroll
        for (int i = 0; i < 4; ++i) *reinterpret_cast<u32x4 *>(base + a_dst[i]) = areg[i];
        const uint32_t words[4] = {wreg.x, wreg.y, wreg.z, wreg.w};
        uint32_t out[16];
#pragma unroll
        for (int blk = 0; blk < 2; ++blk) {
            const float s = blk ? __builtin_amdgcn_cvt_f32_fp8((int)sreg, 1) : __builtin_amdgcn_cvt_f32_fp8((int)sreg, 0);
#pragma unroll
            for (int b = 0; b < 8; ++b) {
                const uint32_t w = words[blk * 2 + (b >> 2)];
                f32x2 v;
                switch (b & 3) {
                    case 0: v = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(w, 1.0f, 0); break;
                    case 1: v = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(w, 1.0f, 1); break;
                    case 2: v = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(w, 1.0f, 2); break;
                    default: v = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(w, 1.0f, 3); break;
                }
                out[blk * 8 + b] = pack_upper_halves(v.x * s, v.y * s);
            }
        }
        u32x4 *dst = reinterpret_cast<u32x4 *>(base + A_BYTES + w_row * PITCH + w_half * 64);
#pragma unroll
        for (int q = 0; q < 4; ++q) dst[q] = u32x4{out[4 * q], out[4 * q + 1], out[4 * q + 2], out[4 * q + 3]};
    };

    const f32x16 zero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
    f32x16 acc[2][2] = {{zero, zero}, {zero, zero}};

    issue(chunk0);
    commit(stage);
    __syncthreads();
    for (int chunk = chunk0; chunk < chunk1; ++chunk) {
        const uint8_t *cur = stage + ((chunk - chunk0) & 1) * STAGE_BYTES;
        if (chunk + 1 < chunk1) issue(chunk + 1);
        const uint8_t *arow = cur + (wm * 64 + l32) * PITCH + half * 16;
        const uint8_t *brow = cur + A_BYTES + (wn * 64 + l32) * PITCH + half * 16;
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) {
            bf16x8 a[2], b[2];
#pragma unroll
            for (int blk = 0; blk < 2; ++blk) {
                a[blk] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const u32x4 *>(arow + blk * 32 * PITCH + ks * 32));
                b[blk] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const u32x4 *>(brow + blk * 32 * PITCH + ks * 32));
            }
#pragma unroll
            for (int mb = 0; mb < 2; ++mb)
#pragma unroll
                for (int nb = 0; nb < 2; ++nb)
                    acc[mb][nb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[mb], b[nb], acc[mb][nb], 0, 0, 0);
        }
        if (chunk + 1 < chunk1) commit(stage + ((chunk + 1 - chunk0) & 1) * STAGE_BYTES);
        __syncthreads();
    }

    const bool direct = L.ksplit == 1;
    if (direct && rejected(L)) return;
    float __attribute__((address_space(1))) *out =
        (float __attribute__((address_space(1))) *)(uintptr_t)(direct ? L.ys
                                                                      : L.partials + (size_t)split * L.tokens * L.rows);
    const float factor = direct ? L.out_scale : 1.0f;
#pragma unroll
    for (int mb = 0; mb < 2; ++mb)
#pragma unroll
        for (int nb = 0; nb < 2; ++nb) {
            const int row = wn * 64 + nb * 32 + l32;
            if (row >= rows_here) continue;
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                const int tok = wm * 64 + mb * 32 + (i >> 2) * 8 + half * 4 + (i & 3);
                if (tok < toks_here) out[(size_t)(tok0 + tok) * L.rows + row0 + row] = acc[mb][nb][i] * factor;
            }
        }
}

// ys = out_scale * (partial 0 + partial 1 + ...), added in split order
__global__ __launch_bounds__(256) void fp4_split_sum_kernel(const Fp4MfmaLaunch L, size_t n) {
    if (rejected(L)) return;
    const float *__restrict__ partials = L.partials;
    float *__restrict__ ys = L.ys;
    const int ksplit = L.ksplit;
    const float out_scale = L.out_scale;
    const size_t i = ((size_t)blockIdx.x * 256 + threadIdx.x) * 4;
    if (i >= n) return;
    if ((n & 3) == 0) {
        float4 sum = *reinterpret_cast<const float4 *>(partials + i);
        for (int s = 1; s < ksplit; ++s) {
            const float4 p = *reinterpret_cast<const float4 *>(partials + (size_t)s * n + i);
            sum.x += p.x; sum.y += p.y; sum.z += p.z; sum.w += p.w;
        }
        ys[i] = sum.x * out_scale; ys[i + 1] = sum.y * out_scale; ys[i + 2] = sum.z * out_scale;
        ys[i + 3] = sum.w * out_scale;
    } else {
        for (size_t j = i; j < n && j < i + 4; ++j) {
            float sum = partials[j];
            for (int s = 1; s < ksplit; ++s) sum += partials[(size_t)s * n + j];
            ys[j] = sum * out_scale;
        }
    }
}

}  // namespace

int fp4_mfma_splits(int rows, int cols, int tokens) {
    const int tiles = ((tokens + TM - 1) / TM) * ((rows + TN - 1) / TN);
    const int chunks = cols / KC;
    int splits = (512 + tiles - 1) / tiles;            // aim at two workgroups per compute unit
    if (splits > 8) splits = 8;
    if (splits > chunks / 4) splits = chunks / 4;      // at least four chunks per split
    // with chunks shared out in equal runs the last split must still own one (30 chunks in 7 splits of 5 would not)
    while (splits > 1 && (splits - 1) * ((chunks + splits - 1) / splits) >= chunks) --splits;
    return splits < 1 ? 1 : splits;
}

int fp4_mfma_launch(const Fp4MfmaLaunch &L, hipStream_t stream) {
    if (L.rows < 1 || L.tokens < 1 || L.cols < KC || (L.cols % KC) || L.ksplit < 1) return -1;
    if (L.flags ? (L.nflags < 1 || !L.outcome) : !L.status) return -1;
    Geometry G;
    G.m_tiles = (L.tokens + TM - 1) / TM;
    G.n_tiles = (L.rows + TN - 1) / TN;
    G.chunks = L.cols / KC;
    G.chunks_per_split = (G.chunks + L.ksplit - 1) / L.ksplit;
    if ((L.ksplit - 1) * G.chunks_per_split >= G.chunks) return -1;        // every split owns a chunk
    if (L.ksplit > 1 && !L.partials) return -1;
    const long long grid = (long long)G.m_tiles * G.n_tiles * L.ksplit;
    if (grid > 0x7FFFFFFFLL) return -1;
    hipLaunchKernelGGL(fp4_mfma_kernel, dim3((unsigned)grid), dim3(256), 0, stream, L, G);
    if (L.ksplit > 1) {
        const size_t n = (size_t)L.tokens * L.rows;
        hipLaunchKernelGGL(fp4_split_sum_kernel, dim3((unsigned)((n / 4 + 256) / 256)), dim3(256), 0, stream, L, n);
    }
    return hipGetLastError() == hipSuccess ? 0 : -1;
}

}  // namespace mi355
