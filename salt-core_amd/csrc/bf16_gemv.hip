// bf16 matrix times fp32 vector in the reference's eight-chain order (the language-model head and the tied
// embedding, reference src/kernels.c:139-174 and src/gpu_hip.cpp:1308-1341).
//
// Row r:   a[j] accumulates the columns c with c % 8 == j, left to right, every product and every sum rounded
// separately;  s = ((a0 + a2) + (a4 + a6)) + ((a1 + a3) + (a5 + a7));  columns past the last multiple of eight are
// added to s in order;  y[r] = s + (bias ? bias[r] : 0.0f).
//
// The matrix is streamed once: a wave owns 64 rows (lane = row) and walks them in chunks of 64 columns.  A chunk is
// 64 rows x 128 bytes; the wave fetches it straight into LDS with eight 16-byte-per-lane loads whose addresses are
// contiguous per row, and each lane then reads its own row back with 16-byte LDS reads.  Several chunks per wave
// are in flight, so LDS is also the latency buffer and no vector registers are held by loads.  The 16-byte
// segments of a row are stored at an exclusive-or of the segment number with bits of the row number, which puts the
// sixteen lanes of one LDS read phase on sixteen different bank groups.  Activations are wave-uniform and arrive as
// scalar operands.
#include "mi355_internal.h"

namespace mi355 {
namespace {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef const u32x4 __attribute__((address_space(1))) *global_u128_ptr;
typedef const float __attribute__((address_space(4))) *uniform_f32_ptr;
typedef __attribute__((address_space(3))) void *lds_void_ptr;

constexpr int ROWS = 64;            // rows per wave
constexpr int CHUNK = 64;           // columns per chunk: 8 segments of 8 columns (16 bytes)
constexpr int SLOTS = ROWS * 8;     // 16-byte slots per stage
constexpr int STREAMING = 2;        // cache policy of the matrix loads: non-temporal (every byte is read once);
                                    // measured 6.9 TB/s against 6.1 TB/s with the default policy

__device__ __forceinline__ int swizzle(int row) { return (row >> 1) & 7; }

template <int PENDING>
__device__ __forceinline__ void wait_loads() {
    // vmcnt counts the direct-to-LDS loads still outstanding
    if (PENDING == 0) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    else if (PENDING == 8) asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
    else if (PENDING == 16) asm volatile("s_waitcnt vmcnt(16)" ::: "memory");
    else if (PENDING == 24) asm volatile("s_waitcnt vmcnt(24)" ::: "memory");
    else if (PENDING == 32) asm volatile("s_waitcnt vmcnt(32)" ::: "memory");
    else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
}

// NB activation rows (1 or 2), STAGES chunks of LDS per wave, WAVES independent waves per workgroup.
template <int NB, int STAGES, int WAVES>
__global__ __launch_bounds__(WAVES * 64) void bf16_tile_kernel(Bf16Launch L) {
    static_assert(STAGES >= 2 && STAGES <= 5, "the wait below knows up to four chunks in flight");
    __shared__ u32x4 lds[WAVES][STAGES][SLOTS];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int tile = blockIdx.x * WAVES + wave;
    const int row0 = tile * ROWS;
    if (row0 >= L.rows) return;
    const int rows_here = L.rows - row0 < ROWS ? L.rows - row0 : ROWS;
    const int C = L.cols;
    const int nchunk = (C + CHUNK - 1) / CHUNK;
    const int tail_segs = (C % CHUNK) / 8;           // segments of the last chunk when it is partial
    u32x4 *mine = &lds[wave][0][0];

    const uint8_t *tile_base = (const uint8_t *)L.weights + (size_t)row0 * C * 2;
    // load k of a chunk covers rows 8k..8k+7; lane i lands in slot 64k + i = row (8k + i/8), position i % 8
    uint32_t src_off[8], src_off_tail[8];
#pragma unroll
    for (int k = 0; k < 8; ++k) {
        int row = k * 8 + (lane >> 3);
        const int seg = (lane & 7) ^ swizzle(row);
        row = row < rows_here ? row : rows_here - 1;
        src_off[k] = (uint32_t)row * (uint32_t)C * 2u + (uint32_t)seg * 16u;
        const int tseg = tail_segs == 0 ? seg : (seg < tail_segs ? seg : tail_segs - 1);
        src_off_tail[k] = (uint32_t)row * (uint32_t)C * 2u + (uint32_t)tseg * 16u;
    }
    auto issue = [&](int ck) {
        const uint8_t *base = tile_base + (size_t)ck * (CHUNK * 2);
        u32x4 *stage = mine + (ck % STAGES) * SLOTS;
        const bool partial = tail_segs != 0 && ck == nchunk - 1;
#pragma unroll
        for (int k = 0; k < 8; ++k) {
            const uint32_t off = partial ? src_off_tail[k] : src_off[k];
            __builtin_amdgcn_global_load_lds((global_u128_ptr)(uintptr_t)(base + off), (lds_void_ptr)(stage + k * 64), 16,
                                             0, STREAMING);
        }
    };

    // slot of this lane's row for segment s: lane * 8 + (s ^ swizzle(lane))
    const int my_swz = swizzle(lane);
    float acc[NB][8];
#pragma unroll
    for (int t = 0; t < NB; ++t)
#pragma unroll
        for (int j = 0; j < 8; ++j) acc[t][j] = 0.0f;

    const uniform_f32_ptr xbase = (uniform_f32_ptr)(uintptr_t)L.x;

    // Activations of XS segments (for all NB rows at most 64 scalar registers) are requested together, so one wait
    // covers them instead of one wait per segment.
    constexpr int XS = NB == 1 ? 8 : 4;
    auto consume = [&](int ck, int segs) {
        const u32x4 *stage = mine + (ck % STAGES) * SLOTS + lane * 8;
        const uniform_f32_ptr xc = xbase + (size_t)ck * CHUNK;
#pragma unroll
        for (int s0 = 0; s0 < 8; s0 += XS) {
            if (s0 >= segs) break;
            float xq[NB][XS * 8];
#pragma unroll
            for (int t = 0; t < NB; ++t)
#pragma unroll
                for (int k = 0; k < XS * 8; ++k)
                    if (s0 * 8 + k < segs * 8) xq[t][k] = xc[(size_t)t * L.x_stride + s0 * 8 + k];
#pragma unroll
            for (int s = s0; s < s0 + XS; ++s) {
                if (s >= segs) break;
                const u32x4 v = stage[s ^ my_swz];
                const uint32_t word[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
                for (int t = 0; t < NB; ++t)
#pragma unroll
                    for (int p = 0; p < 4; ++p) {
                        const float lo = __uint_as_float(word[p] << 16), hi = __uint_as_float(word[p] & 0xffff0000u);
                        acc[t][2 * p] = acc[t][2 * p] + lo * xq[t][(s - s0) * 8 + 2 * p];
                        acc[t][2 * p + 1] = acc[t][2 * p + 1] + hi * xq[t][(s - s0) * 8 + 2 * p + 1];
                    }
            }
        }
    };

#pragma unroll
    for (int st = 0; st < STAGES - 1; ++st)
        if (st < nchunk) issue(st);
    for (int ck = 0; ck < nchunk; ++ck) {
        // the stage written next was read in the previous iteration: those reads have returned before the loads go out
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        if (ck + STAGES - 1 < nchunk) {
            issue(ck + STAGES - 1);
            wait_loads<8 * (STAGES - 1)>();
        } else {
            wait_loads<0>();
        }
        const int segs = (tail_segs != 0 && ck == nchunk - 1) ? tail_segs : 8;
        if (segs == 8) consume(ck, 8);
        else consume(ck, segs);
    }

    if (lane < rows_here) {
        const int row = row0 + lane;
        const float bias = L.bias ? L.bias[row] : 0.0f;
#pragma unroll
        for (int t = 0; t < NB; ++t) {
            const float *a = acc[t];
            const float s = ((a[0] + a[2]) + (a[4] + a[6])) + ((a[1] + a[3]) + (a[5] + a[7]));
            L.y[(size_t)t * L.y_stride + row] = s + bias;
        }
    }
}

// Any column count and any weight address: one thread per row, two-byte loads.
__global__ __launch_bounds__(64) void bf16_generic_kernel(Bf16Launch L) {
    const int row = blockIdx.x * 64 + threadIdx.x;
    if (row >= L.rows) return;
    const uint8_t *w = (const uint8_t *)L.weights + (size_t)row * L.cols * 2;
    auto weight = [&](int c) { return __uint_as_float(((uint32_t)w[2 * c] | ((uint32_t)w[2 * c + 1] << 8)) << 16); };
    const float bias = L.bias ? L.bias[row] : 0.0f;
    for (int t = 0; t < L.tokens; ++t) {
        const float *x = L.x + (size_t)t * L.x_stride;
        float a[8] = {0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f};
        int c = 0;
        for (; c + 7 < L.cols; c += 8)
#pragma unroll
            for (int j = 0; j < 8; ++j) a[j] = a[j] + weight(c + j) * x[c + j];
        float s = ((a[0] + a[2]) + (a[4] + a[6])) + ((a[1] + a[3]) + (a[5] + a[7]));
        for (; c < L.cols; ++c) s = s + weight(c) * x[c];
        L.y[(size_t)t * L.y_stride + row] = s + bias;
    }
}

template <int NB, int STAGES, int WAVES>
void launch_tiles(const Bf16Launch &L, hipStream_t stream) {
    const int tiles = (L.rows + ROWS - 1) / ROWS;
    bf16_tile_kernel<NB, STAGES, WAVES><<<dim3((tiles + WAVES - 1) / WAVES), dim3(WAVES * 64), 0, stream>>>(L);
}

// two stages, four waves per workgroup: 64 KB of LDS, eight waves per compute unit (measured best of
// {2,1} {3,1} {2,2} {2,4} stages x waves on the 262144 x 2816 head)
template <int NB>
void launch_shape(const Bf16Launch &L, hipStream_t stream) { launch_tiles<NB, 2, 4>(L, stream); }

}  // namespace

bool bf16_is_tileable(const Bf16Launch &L) {
    return L.cols >= 8 && L.cols % 8 == 0 && ((uintptr_t)L.weights & 15) == 0 && ((uintptr_t)L.x & 3) == 0 &&
           (uint64_t)ROWS * (uint64_t)L.cols * 2u < (1ull << 32);
}

int bf16_launch(const Bf16Launch &L, hipStream_t stream) {
    if (!L.weights || !L.x || !L.y || L.rows < 1 || L.cols < 1 || L.tokens < 1) return -1;
    if (!bf16_is_tileable(L)) {
        bf16_generic_kernel<<<dim3((L.rows + 63) / 64), dim3(64), 0, stream>>>(L);
        return hipGetLastError() == hipSuccess ? 0 : -1;
    }
    // two activation rows per pass: the pass stays bound by the matrix stream, which wider passes do not
    for (int first = 0; first < L.tokens; first += 2) {
        Bf16Launch part = L;
        part.x = L.x + (size_t)first * L.x_stride;
        part.y = L.y + (size_t)first * L.y_stride;
        part.tokens = L.tokens - first < 2 ? L.tokens - first : 2;
        if (part.tokens == 1) launch_shape<1>(part, stream);
        else launch_shape<2>(part, stream);
        if (hipGetLastError() != hipSuccess) return -1;
    }
    return 0;
}

}  // namespace mi355
