// NVFP4 matvec and activation quantise/dequantise for gfx950, bit-identical to
// the engine's CPU reference (reference src/nvfp4.c).
//
// Weight element (reference nvfp4.c:173-192):
//     scaled = fl(e4m3(scale[row][col/16]) * weight_global_scale)
//     w      = fl(e2m1(code) * scaled);  p = fl(w * x[col]);  acc[col%32] += p
// with the same 32 chains and the same fold as the affine-Q4 row.  The matvec
// kernel has the Q4 kernel's shape (lane = row, wave-uniform chain slice,
// scalar-loaded activations, LDS-staged codes, in-order fold); only decoding
// differs: v_cvt_scalef32_pk_f32_fp4 turns one byte into two E2M1 values
// without any masking, and the per-16-column `scaled` factors are produced
// once per tile step into LDS with the hardware E4M3 decoder.
//
// E2M1 code 8 ("-0") decodes to +0 in the reference and to -0 in hardware.
// The difference never reaches a result: it only flips the sign of a zero
// product, and a chain accumulator that starts at +0 can never become -0.
//
// The activation pre-pass (reference nvfp4.c:82-130) runs one thread per
// 16-element block with closed-form round-to-nearest-even encoders in place of
// the reference's argmin scans (equality is proven on the host by the tests).
#include "mi355_internal.h"
#include "nvfp4_device.h"

#include <stddef.h>

namespace mi355 {
namespace {

typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef const float __attribute__((address_space(4))) *uniform_f32_ptr;
typedef const uint64_t __attribute__((address_space(4))) *uniform_u64_ptr;
typedef const uint8_t __attribute__((address_space(1))) *global_u8_ptr;
typedef const uint16_t __attribute__((address_space(1))) *global_u16_ptr;
typedef u32x4 __attribute__((aligned(4))) u32x4_dword_aligned;       // 128-bit global loads need dword alignment only
typedef const u32x4_dword_aligned __attribute__((address_space(1))) *global_u128_ptr;
typedef float __attribute__((address_space(1))) *global_f32_out_ptr;

constexpr int TILE_ROWS = 64;
constexpr int CHUNK_BLOCKS = 16;                       // 32-column blocks per staged step
constexpr int W_PITCH = 16 * CHUNK_BLOCKS + 4;         // bytes per staged row of codes
constexpr int M_PITCH = 2 * CHUNK_BLOCKS + 1;          // floats per staged row of `scaled` factors (odd)
constexpr int W_STAGE = TILE_ROWS * W_PITCH;
constexpr int M_STAGE = TILE_ROWS * M_PITCH;
constexpr int FOLD_PITCH = 33;

static_assert(sizeof(Fp4Job) == 48 && offsetof(Fp4Job, weight_global_scale) == 32 && offsetof(Fp4Job, rows) == 36 &&
              offsetof(Fp4Job, tile0) == 40 && offsetof(Fp4Job, x_stride) == 44,
              "find_job reads a job record as six 64-bit words");

__device__ __forceinline__ Fp4Job find_job(const Fp4Launch &L, int tile) {
    if (L.table == nullptr) return L.one;
    const uniform_u64_ptr words = (uniform_u64_ptr)(uintptr_t)L.table;     // 6 words per record
    int lo = 0, hi = L.njobs - 1;
    while (lo < hi) {
        const int mid = (lo + hi + 1) >> 1;
        if ((int)(uint32_t)words[6 * mid + 5] <= tile) lo = mid; else hi = mid - 1;
    }
    const uniform_u64_ptr rec = words + 6 * lo;
    Fp4Job job;
    job.packed = (const uint8_t *)rec[0];
    job.scales = (const uint8_t *)rec[1];
    job.x = (const float *)rec[2];
    job.y = (float *)rec[3];
    job.weight_global_scale = __uint_as_float((uint32_t)rec[4]);
    job.rows = (int)(rec[4] >> 32);
    job.tile0 = (int)(uint32_t)rec[5];
    job.x_stride = (int)(rec[5] >> 32);
    return job;
}

// Quantise and dequantise one 16-element block (reference nvfp4.c:82-130).
// Returns false when an element is not finite (the reference rejects the call).
__device__ __forceinline__ bool qdq_block(const float (&v)[16], float g, uint32_t &scale_code, uint32_t (&bytes)[2],
                                          float (&out)[16], uint32_t (&halves)[8]) {
    float top = 0.0f;
    bool finite = true;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
        const float m = __builtin_fabsf(v[i]);
        finite = finite && (m < __builtin_inff());           // false for inf and NaN
        if (m > top) top = m;
    }
    if (!finite) return false;
    const float sixth = top * (1.0f / 6.0f);
    float raw = g * sixth;
    if (raw > 448.0f) raw = 448.0f;
    scale_code = e4m3_encode_positive(raw);
    const float scale = __builtin_amdgcn_cvt_f32_fp8((int)scale_code, 0);
    const float to_code = scale == 0.0f ? 0.0f : g / scale;
    const float from_code = scale / g;
    bytes[0] = 0u; bytes[1] = 0u;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
        float s = v[i] * to_code;
        if (s > 6.0f) s = 6.0f;
        if (s < -6.0f) s = -6.0f;
        const uint32_t code = e2m1_encode(s);
        bytes[i >> 3] |= code << (4 * (i & 7));
        const float value = e2m1_decode(code);
        out[i] = value * from_code;
        // code value * block scale: at most six significant bits, exact in bf16
        const uint32_t h = __float_as_uint(value * scale) >> 16;
        if (i & 1) halves[i >> 1] |= h << 16; else halves[i >> 1] = h;
    }
    return true;
}

constexpr int x_batch_blocks(int S, int NB) {
    const int fit = (S == 8 ? 32 : 64) / (S * NB);
    return fit >= 16 ? 16 : fit >= 8 ? 8 : fit >= 4 ? 4 : fit >= 2 ? 2 : 1;
}

// QDQ: the launch's single token is quantised and dequantised by every
// workgroup in its prologue (the activation pass of the reference matvec,
// nvfp4.c:228-256) into LDS, and the rows read it from there into vector
// registers (every lane the same words); workgroup 0 reports a non-finite activation (-1 into a
// status word the caller cleared) and nothing is published then.
template <int S, int NB, bool QDQ = false>
__global__ __launch_bounds__((32 / S) * 64) void fp4_tile_kernel(const Fp4Launch L) {
    constexpr int WAVES = 32 / S;
    constexpr int THREADS = WAVES * 64;
    constexpr int PIECES = (TILE_ROWS * CHUNK_BLOCKS) / THREADS;     // 16-byte pieces == (row, block) items
    constexpr int FOLD_BYTES = NB * TILE_ROWS * FOLD_PITCH * 4;
    constexpr int W_BYTES = 2 * W_STAGE > FOLD_BYTES ? 2 * W_STAGE : FOLD_BYTES;
    constexpr int XB = QDQ ? 2 : x_batch_blocks(S, NB);      // LDS-fed activations sit in vector registers: short batches
    constexpr int XN = XB * S;
    constexpr int W_ROW_STEP = THREADS / 16;
    static_assert(THREADS >= NB * TILE_ROWS, "fold needs one thread per (token, row)");

    __shared__ __attribute__((aligned(16))) uint8_t w_lds[W_BYTES];
    __shared__ float m_lds[2 * M_STAGE];
    __shared__ __attribute__((aligned(16))) float x_lds[QDQ ? FP4_FUSED_MAX_COLS : 4];
    __shared__ int x_bad;
    static_assert(!QDQ || NB == 1, "the fused activation pass serves single-token launches");

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);

    const Fp4Job job = find_job(L, blockIdx.x);
    if (QDQ) {
        if (tid == 0) x_bad = 0;
        __syncthreads();
        for (int blk = tid; blk < (L.cols >> 4); blk += THREADS) {
            const float4 *src = reinterpret_cast<const float4 *>(job.x + (size_t)blk * 16);
            float v[16];
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const float4 f = src[q];
                v[4 * q] = f.x; v[4 * q + 1] = f.y; v[4 * q + 2] = f.z; v[4 * q + 3] = f.w;
            }
            uint32_t scale_code, bytes[2], halves[8];
            float out[16];
            if (!qdq_block(v, L.input_global_scale, scale_code, bytes, out, halves)) { x_bad = 1; continue; }
            float4 *dst = reinterpret_cast<float4 *>(x_lds + blk * 16);
#pragma unroll
            for (int q = 0; q < 4; ++q) dst[q] = make_float4(out[4 * q], out[4 * q + 1], out[4 * q + 2], out[4 * q + 3]);
        }
        __syncthreads();
        const int bad = x_bad;
        if (bad && blockIdx.x == 0 && tid == 0) *L.status = -1;        // like fp4_qdq_kernel: the caller cleared it
        if (bad) return;                                   // uniform
    }
    const int row0 = (blockIdx.x - job.tile0) * TILE_ROWS;
    const int rows_here = job.rows - row0 < TILE_ROWS ? job.rows - row0 : TILE_ROWS;
    const int nblk = L.cols >> 5;
    const int nchunk = (nblk + CHUNK_BLOCKS - 1) / CHUNK_BLOCKS;
    const uint32_t row_bytes = (uint32_t)(L.cols >> 1);
    const uint32_t row_pairs = (uint32_t)nblk;                       // scale byte pairs per row
    const global_u8_ptr codes = (global_u8_ptr)(uintptr_t)job.packed + (size_t)row0 * row_bytes;
    const global_u16_ptr scale_pairs = (global_u16_ptr)(uintptr_t)job.scales + (size_t)row0 * row_pairs;
    const global_f32_out_ptr y = (global_f32_out_ptr)(uintptr_t)job.y;
    const uniform_f32_ptr xbase = (uniform_f32_ptr)(uintptr_t)job.x + S * wave;
    const float wg = job.weight_global_scale;

    // Piece i of a thread: row (tid>>4) + i*W_ROW_STEP, block column tid&15.
    // The same (row, block) item also owns that block's two scale bytes.
    const uint32_t seg = tid & 15;
    const uint32_t w_dst0 = (tid >> 4) * W_PITCH + seg * 16;
    const uint32_t m_dst0 = (tid >> 4) * M_PITCH + seg * 2;
    uint32_t src_row[PIECES];
#pragma unroll
    for (int i = 0; i < PIECES; ++i) {
        const int row = (tid >> 4) + i * W_ROW_STEP;
        src_row[i] = (uint32_t)(row < rows_here ? row : rows_here - 1);
    }

    u32x4 wreg[PIECES];
    uint32_t mreg[PIECES];

    auto issue = [&](int ck) {
#pragma unroll
        for (int i = 0; i < PIECES; ++i) {
            int blk = ck * CHUNK_BLOCKS + (int)seg;
            blk = blk < nblk ? blk : nblk - 1;
            wreg[i] = __builtin_nontemporal_load((global_u128_ptr)(codes + (src_row[i] * row_bytes + (uint32_t)blk * 16u)));
            mreg[i] = scale_pairs[src_row[i] * row_pairs + (uint32_t)blk];
        }
    };
    auto commit = [&](int stage) {
#pragma unroll
        for (int i = 0; i < PIECES; ++i) {
            uint32_t *dst = reinterpret_cast<uint32_t *>(w_lds + stage * W_STAGE + w_dst0 + i * W_ROW_STEP * W_PITCH);
            dst[0] = wreg[i].x; dst[1] = wreg[i].y; dst[2] = wreg[i].z; dst[3] = wreg[i].w;
            float *m = m_lds + stage * M_STAGE + m_dst0 + i * W_ROW_STEP * M_PITCH;
            m[0] = __builtin_amdgcn_cvt_f32_fp8((int)mreg[i], 0) * wg;      // columns 0..15 of the block
            m[1] = __builtin_amdgcn_cvt_f32_fp8((int)mreg[i], 1) * wg;      // columns 16..31
        }
    };

    float acc[NB][S];
#pragma unroll
    for (int t = 0; t < NB; ++t)
#pragma unroll
        for (int c = 0; c < S; ++c) acc[t][c] = 0.0f;

    issue(0);

    auto load_x = [&](int blk0, float (&xq)[NB][XN], int blocks) {
        if (QDQ) {                        // every lane reads the same LDS words: the activations travel in vector registers
            const float *xl = x_lds + blk0 * 32 + S * wave;
#pragma unroll
            for (int k = 0; k < XN; ++k)
                if (k < blocks * S) xq[0][k] = xl[(k / S) * 32 + (k % S)];
            return;
        }
        const uniform_f32_ptr xg = xbase + (size_t)blk0 * 32;
#pragma unroll
        for (int t = 0; t < NB; ++t)
#pragma unroll
            for (int k = 0; k < XN; ++k)
                if (k < blocks * S) xq[t][k] = xg[(size_t)t * job.x_stride + (k / S) * 32 + (k % S)];
    };

    // One block of one lane: S codes against the wave's S chains.
    auto consume = [&](uint32_t w, float scaled, const float (&xq)[NB][XN], int xat) {
#pragma unroll
        for (int b = 0; b < S / 2; ++b) {
            f32x2 v;
            switch (b) {                       // the byte selector is an immediate
                case 0: v = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(w, 1.0f, 0); break;
                case 1: v = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(w, 1.0f, 1); break;
                case 2: v = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(w, 1.0f, 2); break;
                default: v = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(w, 1.0f, 3); break;
            }
            const float w0 = v.x * scaled, w1 = v.y * scaled;
#pragma unroll
            for (int t = 0; t < NB; ++t) {
                const float p0 = w0 * xq[t][xat + 2 * b];
                acc[t][2 * b] = acc[t][2 * b] + p0;
                const float p1 = w1 * xq[t][xat + 2 * b + 1];
                acc[t][2 * b + 1] = acc[t][2 * b + 1] + p1;
            }
        }
    };

    for (int ck = 0; ck < nchunk; ++ck) {
        const int stage = ck & 1;
        const int remaining = nblk - ck * CHUNK_BLOCKS;
        const bool full = remaining >= CHUNK_BLOCKS;
        const int bcount = full ? CHUNK_BLOCKS : remaining;

        float xq[NB][XN];
        if (full) load_x(ck * CHUNK_BLOCKS, xq, XB);

        commit(stage);
        __syncthreads();
        if (ck + 1 < nchunk) issue(ck + 1);

        const uint8_t *wrow = w_lds + stage * W_STAGE + lane * W_PITCH + wave * (S / 2);
        // the wave's chains lie in the first (columns 0..15) or second half of a block
        const float *mrow = m_lds + stage * M_STAGE + lane * M_PITCH + ((S * wave) >> 4);

        auto fetch = [&](int blk, uint32_t &w, float &scaled) {
            scaled = mrow[2 * blk];
            if (S == 8) w = *reinterpret_cast<const uint32_t *>(wrow + blk * 16);
            else if (S == 4) w = *reinterpret_cast<const uint16_t *>(wrow + blk * 16);
            else w = wrow[blk * 16];
        };

        if (full) {
#pragma unroll
            for (int batch = 0; batch < CHUNK_BLOCKS / XB; ++batch) {
                if (batch > 0) load_x(ck * CHUNK_BLOCKS + batch * XB, xq, XB);
#pragma unroll
                for (int bl = 0; bl < XB; ++bl) {
                    uint32_t w;
                    float scaled;
                    fetch(batch * XB + bl, w, scaled);
                    consume(w, scaled, xq, bl * S);
                }
            }
        } else {
            for (int blk = 0; blk < bcount; ++blk) {
                uint32_t w;
                float scaled;
                fetch(blk, w, scaled);
                load_x(ck * CHUNK_BLOCKS + blk, xq, 1);
                consume(w, scaled, xq, 0);
            }
        }
    }

    __syncthreads();
    float *fold = reinterpret_cast<float *>(w_lds);
#pragma unroll
    for (int t = 0; t < NB; ++t)
#pragma unroll
        for (int c = 0; c < S; ++c) fold[(t * TILE_ROWS + lane) * FOLD_PITCH + S * wave + c] = acc[t][c];
    __syncthreads();
    if (tid < NB * TILE_ROWS) {
        const int t = tid >> 6;
        const float *f = fold + (t * TILE_ROWS + lane) * FOLD_PITCH;
        float part[4] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int a = 0; a < 8; ++a)
#pragma unroll
            for (int j = 0; j < 4; ++j) part[j] = part[j] + f[4 * a + j];
        const float even = part[0] + part[2];
        const float odd = part[1] + part[3];
        if (lane < rows_here) y[(size_t)t * job.rows + row0 + lane] = even + odd;
    }
}

template <int S>
int launch_tiles(const Fp4Launch &L, hipStream_t stream) {
    const dim3 grid(L.total_tiles), block((32 / S) * 64);
    if (L.qdq) {
        if (L.tokens != 1 || L.table || L.cols > FP4_FUSED_MAX_COLS || !L.status || ((uintptr_t)L.one.x & 15)) return -1;
        hipLaunchKernelGGL((fp4_tile_kernel<S, 1, true>), grid, block, 0, stream, L);
        return hipGetLastError() == hipSuccess ? 0 : -1;
    }
    switch (L.tokens) {
        case 1: hipLaunchKernelGGL((fp4_tile_kernel<S, 1>), grid, block, 0, stream, L); break;
        case 2: hipLaunchKernelGGL((fp4_tile_kernel<S, 2>), grid, block, 0, stream, L); break;
        case 3: hipLaunchKernelGGL((fp4_tile_kernel<S, 3>), grid, block, 0, stream, L); break;
        case 4: hipLaunchKernelGGL((fp4_tile_kernel<S, 4>), grid, block, 0, stream, L); break;
        default: return -1;
    }
    return hipGetLastError() == hipSuccess ? 0 : -1;
}

// ---------------------------------------------------------------- activation Q/DQ

// One thread per 16-element block of one token.  FLAGS: the workgroup reports in flags[blockIdx.x] (0 or -1, always
// written) instead of setting *status.
template <bool FLAGS>
__global__ __launch_bounds__(256) void fp4_qdq_kernel(const float *__restrict__ input, int cols, int tokens,
                                                      float g, uint8_t *__restrict__ packed,
                                                      uint8_t *__restrict__ scales, float *__restrict__ dequant,
                                                      uint16_t *__restrict__ plane, int *__restrict__ status) {
    const int blocks_per_token = cols >> 4;
    const long long item = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    const bool present = item < (long long)blocks_per_token * tokens;
    if (!FLAGS && !present) return;
    float v[16];
#pragma unroll
    for (int q = 0; q < 16; ++q) v[q] = 0.0f;
    if (present) {
        const float4 *src = reinterpret_cast<const float4 *>(input + item * 16);
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const float4 f = src[q];
            v[4 * q] = f.x; v[4 * q + 1] = f.y; v[4 * q + 2] = f.z; v[4 * q + 3] = f.w;
        }
    }
    uint32_t scale_code, bytes[2], halves[8];
    float out[16];
    const bool good = qdq_block(v, g, scale_code, bytes, out, halves);    // the reference rejects the whole call
    if (FLAGS) {
        const int any_bad = __syncthreads_or(good ? 0 : 1);
        if (threadIdx.x == 0) status[blockIdx.x] = any_bad ? -1 : 0;
        if (!present || !good) return;
    } else if (!good) {
        *status = -1;
        return;
    }
    if (scales) scales[item] = (uint8_t)scale_code;
    if (packed) reinterpret_cast<uint2 *>(packed)[item] = make_uint2(bytes[0], bytes[1]);
    if (dequant) {
        float4 *dst = reinterpret_cast<float4 *>(dequant + item * 16);
#pragma unroll
        for (int q = 0; q < 4; ++q) dst[q] = make_float4(out[4 * q], out[4 * q + 1], out[4 * q + 2], out[4 * q + 3]);
    }
    if (plane) {
        uint4 *dst = reinterpret_cast<uint4 *>(plane + item * 16);
        dst[0] = make_uint4(halves[0], halves[1], halves[2], halves[3]);
        dst[1] = make_uint4(halves[4], halves[5], halves[6], halves[7]);
    }
}

}  // namespace

int fp4_launch(const Fp4Launch &L, int chains_per_lane, hipStream_t stream) {
    if (L.total_tiles < 1 || L.tokens < 1 || L.tokens > 4 || L.cols < 32 || (L.cols & 31)) return -1;
    int S = chains_per_lane;
    // as for the affine-Q4 kernel: sixteen waves per tile up to one tile per compute unit, eight beyond (8192 columns,
    // one token: 23.9 against 30.2 us at 256 tiles, 42.5 against 36.0 at 320, 48.5 against 43.8 at 512)
    if (S == 0) S = L.total_tiles > 256 ? 4 : 2;
    switch (S) {
        case 8: return launch_tiles<8>(L, stream);
        case 4: return launch_tiles<4>(L, stream);
        case 2: return launch_tiles<2>(L, stream);
        default: return -1;
    }
}

int fp4_qdq_launch(const float *input, int cols, int tokens, float input_global_scale, uint8_t *packed,
                   uint8_t *scales, float *dequant, uint16_t *plane, int *status, hipStream_t stream) {
    const long long items = (long long)(cols >> 4) * tokens;
    if (items < 1 || (cols & 15)) return -1;
    const unsigned grid = (unsigned)((items + 255) / 256);
    hipLaunchKernelGGL(fp4_qdq_kernel<false>, dim3(grid), dim3(256), 0, stream, input, cols, tokens, input_global_scale,
                       packed, scales, dequant, plane, status);
    return hipGetLastError() == hipSuccess ? 0 : -1;
}

int fp4_qdq_flag_count(int cols, int tokens) {
    const long long items = (long long)(cols >> 4) * tokens;
    return items < 1 || items > (1ll << 38) ? 0 : (int)((items + 255) / 256);
}

int fp4_qdq_flags_launch(const float *input, int cols, int tokens, float input_global_scale, uint16_t *plane,
                         int *flags, hipStream_t stream) {
    const int grid = fp4_qdq_flag_count(cols, tokens);
    if (grid < 1 || (cols & 15) || !flags) return -1;
    hipLaunchKernelGGL(fp4_qdq_kernel<true>, dim3((unsigned)grid), dim3(256), 0, stream, input, cols, tokens,
                       input_global_scale, (uint8_t *)nullptr, (uint8_t *)nullptr, (float *)nullptr, plane, flags);
    return hipGetLastError() == hipSuccess ? 0 : -1;
}

}  // namespace mi355
