// The fp32 cells around the MoE step of a decoder layer: RMS norm, router input, residual post-norm, parallel
// feed-forward combine, softcap (reference models/gemma4-26b-a4b/src/gemma4.c:46-130, 188-286; the backend ABI's
// exact cells, include/salt/gpu.h:211-234, src/gpu_hip.cpp:2034-2063, 2389-2458, 2688-2745).
//
// Every norm needs ss = x0*x0 + x1*x1 + ... added left to right in fp32.  The squares are computed by the whole
// workgroup into LDS; one lane then walks them with dependent additions (several vectors at once ride in
// neighbouring lanes of that wave).  inv = pow(ss / n + eps, -0.5) is six double-precision Newton steps from the
// 0x5f3759df seed (src/bitmath.c:114-142).  A cell that meets a non-finite input or result publishes nothing and
// sets the sticky status word to -1; a cell that finds the status word set does nothing.
#include "device_math.h"
#include "mi355_internal.h"

namespace mi355 {
namespace {

constexpr int THREADS = 1024;         // one workgroup per cell: sixteen waves keep enough loads in flight
constexpr int SLOTS = 4;              // elements a thread handles per pass: i = base + tid + k * THREADS
constexpr int SQ_CHUNK = SLOTS * THREADS;   // squares staged per pass of the serial adder
constexpr int SQ_TAIL = 64;           // floats the adder may read (and drop) past the staged squares

__device__ __forceinline__ double inverse_root64(float x) {
    const float seed = __uint_as_float(0x5f3759dfu - (__float_as_uint(x) >> 1));
    double y = (double)seed;
    const double wide = (double)x;
#pragma unroll
    for (int i = 0; i < 6; ++i) {
        const double square = y * y;
        const double half = 0.5 * wide;
        const double step = 1.5 - half * square;
        y = y * step;
    }
    return y;
}

__device__ float det_rsqrtf(float x) {
    if (x != x) return x;
    if (x < 0.0f) return __uint_as_float(0x7fc00000u);
    if (x == 0.0f) return __uint_as_float(0x7f800000u);
    if (x == 1.0f) return 1.0f;
    if (x < 0x1p-126f) {                               // rescaled once: x * 2^24 is a normal number
        const float up = x * 0x1p24f;
        const float root = up == 1.0f ? 1.0f : (float)inverse_root64(up);
        return root * 0x1p12f;
    }
    return (float)inverse_root64(x);
}

__device__ float det_sqrtf(float x) {
    if (x != x) return x;
    if (x < 0.0f) return __uint_as_float(0x7fc00000u);
    if (x == 0.0f || x == 1.0f) return x;
    if (x < 0x1p-126f) {
        const float up = x * 0x1p24f;
        const float root = up == 1.0f ? 1.0f : (float)((double)up * inverse_root64(up));
        return root * 0x1p-12f;
    }
    return (float)((double)x * inverse_root64(x));
}

// salt_powf(x, -0.5f)
__device__ __forceinline__ float pow_minus_half(float x) {
    if (x == 1.0f) return 1.0f;
    if (x > 0.0f) return det_rsqrtf(x);
    return x;
}

// 1 for an infinity or a NaN; an unsigned, so that flags combine with | and no load hides behind a short circuit
__device__ __forceinline__ unsigned nonfinite(float v) { return (__float_as_uint(v) & 0x7f800000u) == 0x7f800000u; }

// Visits the elements [0, n) SLOTS at a time per thread: f(i, k) for the live slots of a pass, all loads of a pass
// being independent of each other.
template <typename F>
__device__ __forceinline__ void each_element(int n, F f) {
    for (int base = 0; base < n; base += SQ_CHUNK) {
#pragma unroll
        for (int k = 0; k < SLOTS; ++k) {
            const int i = base + (int)threadIdx.x + k * THREADS;
            if (i < n) f(i);
        }
    }
}

// acc + mine[0] + mine[1] + ... + mine[count - 1], left to right.  32 values per batch; the next batch is read from
// LDS while the current one is added, unconditionally one batch ahead (what is read past the end is dropped, the
// staging buffers have a tail for it).
__device__ __forceinline__ float add_staged(const float *mine, int count, float acc) {
    const int full = count & ~31, pairs = full & ~63;
    float4 a[8], b[8];
    auto fetch = [&](float4 (&dst)[8], int at) {
#pragma unroll
        for (int k = 0; k < 8; ++k) dst[k] = *(const float4 *)&mine[at + 4 * k];
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
    for (int i = 0; i < pairs; i += 64) {
        fetch(b, i + 32);
        add(a);
        fetch(a, i + 64);
        add(b);
    }
    if (full != pairs) add(a);
    for (int i = full; i < count; ++i) acc = acc + mine[i];
    return acc;
}

// The same sums for at most SQ_CHUNK elements that the threads already hold: val[v][k] is element tid + k * THREADS of
// vector v.
template <int V>
__device__ __forceinline__ void chains_from_registers(const float (&val)[V][SLOTS], int n, float *sq, float *shared,
                                                      float (&ss)[V]) {
    const int tid = threadIdx.x;
#pragma unroll
    for (int v = 0; v < V; ++v)
#pragma unroll
        for (int k = 0; k < SLOTS; ++k) {
            const int i = tid + k * THREADS;
            if (i < n) sq[v * SQ_CHUNK + i] = val[v][k] * val[v][k];
        }
    __syncthreads();
    if (tid < V) shared[tid] = add_staged(sq + tid * SQ_CHUNK, n, 0.0f);
    __syncthreads();
#pragma unroll
    for (int v = 0; v < V; ++v) ss[v] = shared[v];
    __syncthreads();
}

// Serial sums of squares of `vectors` (1 or 2) vectors of n floats: lane v of wave 0 adds vector v's squares left to
// right.  Returns the sums in ss_out[] on every thread; `bad` collects non-finite elements.  sq is LDS scratch of
// vectors * SQ_CHUNK + SQ_TAIL floats, shared of at least `vectors` floats.
__device__ void serial_square_sums(const float *const *x, int vectors, int n, float *sq, float *ss_out, float *shared,
                                   unsigned &bad) {
    const int tid = threadIdx.x;
    float acc = 0.0f;
    for (int base = 0; base < n; base += SQ_CHUNK) {
        const int count = n - base < SQ_CHUNK ? n - base : SQ_CHUNK;
        for (int v = 0; v < vectors; ++v) {
            const float *src = x[v] + base;
#pragma unroll
            for (int k = 0; k < SLOTS; ++k) {
                const int i = tid + k * THREADS;
                if (i < count) {
                    const float value = src[i];
                    bad |= nonfinite(value);
                    sq[v * SQ_CHUNK + i] = value * value;
                }
            }
        }
        __syncthreads();
        if (tid < vectors) acc = add_staged(sq + tid * SQ_CHUNK, count, acc);
        __syncthreads();
    }
    if (tid < vectors) shared[tid] = acc;
    __syncthreads();
    for (int v = 0; v < vectors; ++v) ss_out[v] = shared[v];
    __syncthreads();
}

__device__ __forceinline__ float inverse_from_sum(float ss, int n, float eps) {
    const float mean = ss / (float)n;
    return pow_minus_half(mean + eps);
}

// kind 0: out = (x * inv) [* weight]            weight may be null
// kind 1: out = ((x * inv) * weight) * root     router input
// kind 2: out = residual + (x * inv) * weight   residual post-norm
struct NormArgs {
    const float *x, *weight, *residual;
    float *out;
    int n, kind;
    float eps, root;
    int *status;
};

__global__ __launch_bounds__(THREADS) void norm_cell_kernel(NormArgs a) {
    __shared__ __attribute__((aligned(16))) float sq[SQ_CHUNK + SQ_TAIL];
    __shared__ float shared[4];
    if (*a.status != 0) return;
    unsigned bad = !(a.eps >= 0.0f) || nonfinite(a.eps);
    const float *vec[1] = {a.x};
    float ss;
    serial_square_sums(vec, 1, a.n, sq, &ss, shared, bad);
    const float inv = inverse_from_sum(ss, a.n, a.eps);
    bad |= nonfinite(inv);
    float root = a.root;
    if (a.kind == 1 && !(root > 0.0f)) root = 1.0f / det_sqrtf((float)a.n);
    auto value = [&](int i, unsigned &flag) {
        float y = a.x[i] * inv;
        if (a.weight) { const float w = a.weight[i]; flag |= nonfinite(w); y = y * w; }
        if (a.kind == 1) y = y * root;
        flag |= nonfinite(y);
        if (a.kind == 2) {
            const float r = a.residual[i];
            y = r + y;
            flag |= nonfinite(r) | nonfinite(y);
        }
        return y;
    };
    each_element(a.n, [&](int i) { (void)value(i, bad); });
    if (__syncthreads_or((int)bad)) {
        if (threadIdx.x == 0) *a.status = -1;
        return;
    }
    unsigned ignored = 0;
    each_element(a.n, [&](int i) { a.out[i] = value(i, ignored); });
}

// One pass over the residual for the three vectors a feed-forward block derives from it:
// norm_a = (r * inv) * w1, router_in = ((r * inv) * scale) * root, norm_b = (r * inv) * w2.
struct PreArgs {
    const float *residual, *w1, *w2, *router_scale;
    float *norm_a, *norm_b, *router_in;
    int n;
    float eps;
    int *status;               // written, not only set: this kernel opens the block
};

// n <= SQ_CHUNK: every input is requested once, up front, and lives in registers from then on
__global__ __launch_bounds__(THREADS) void ffn_pre_small_kernel(PreArgs a) {
    __shared__ __attribute__((aligned(16))) float sq[SQ_CHUNK + SQ_TAIL];
    __shared__ float shared[4];
    unsigned bad = !(a.eps >= 0.0f) || nonfinite(a.eps);
    float r[1][SLOTS], w1[SLOTS], w2[SLOTS], rs[SLOTS];
#pragma unroll
    for (int k = 0; k < SLOTS; ++k) {
        const int i = (int)threadIdx.x + k * THREADS;
        const bool live = i < a.n;
        r[0][k] = live ? a.residual[i] : 0.0f;
        w1[k] = live ? a.w1[i] : 0.0f;
        w2[k] = live ? a.w2[i] : 0.0f;
        rs[k] = live ? a.router_scale[i] : 0.0f;
        bad |= nonfinite(r[0][k]) | nonfinite(w1[k]) | nonfinite(w2[k]) | nonfinite(rs[k]);
    }
    float ss[1];
    chains_from_registers<1>(r, a.n, sq, shared, ss);
    const float inv = inverse_from_sum(ss[0], a.n, a.eps);
    bad |= nonfinite(inv);
    const float root = 1.0f / det_sqrtf((float)a.n);
    float na[SLOTS], nb[SLOTS], ri[SLOTS];
#pragma unroll
    for (int k = 0; k < SLOTS; ++k) {
        const float y = r[0][k] * inv;
        na[k] = y * w1[k];
        nb[k] = y * w2[k];
        ri[k] = (y * rs[k]) * root;
        bad |= nonfinite(y) | nonfinite(na[k]) | nonfinite(nb[k]) | nonfinite(ri[k]);
    }
    const bool failed = __syncthreads_or((int)bad);
    if (threadIdx.x == 0) *a.status = failed ? -1 : 0;
    if (failed) return;
#pragma unroll
    for (int k = 0; k < SLOTS; ++k) {
        const int i = (int)threadIdx.x + k * THREADS;
        if (i < a.n) { a.norm_a[i] = na[k]; a.norm_b[i] = nb[k]; a.router_in[i] = ri[k]; }
    }
}

__global__ __launch_bounds__(THREADS) void ffn_pre_kernel(PreArgs a) {
    __shared__ __attribute__((aligned(16))) float sq[SQ_CHUNK + SQ_TAIL];
    __shared__ float shared[4];
    unsigned bad = !(a.eps >= 0.0f) || nonfinite(a.eps);
    const float *vec[1] = {a.residual};
    float ss;
    serial_square_sums(vec, 1, a.n, sq, &ss, shared, bad);
    const float inv = inverse_from_sum(ss, a.n, a.eps);
    bad |= nonfinite(inv);
    const float root = 1.0f / det_sqrtf((float)a.n);
    each_element(a.n, [&](int i) {
        const float y = a.residual[i] * inv, w1 = a.w1[i], w2 = a.w2[i], rs = a.router_scale[i];
        bad |= nonfinite(w1) | nonfinite(w2) | nonfinite(rs) | nonfinite(y) | nonfinite(y * w1) | nonfinite(y * w2) |
               nonfinite((y * rs) * root);
    });
    const bool failed = __syncthreads_or((int)bad);
    if (threadIdx.x == 0) *a.status = failed ? -1 : 0;
    if (failed) return;
    each_element(a.n, [&](int i) {
        const float y = a.residual[i] * inv;
        a.norm_a[i] = y * a.w1[i];
        a.norm_b[i] = y * a.w2[i];
        a.router_in[i] = (y * a.router_scale[i]) * root;
    });
}

// out = (residual + norm(norm(dense) * wd + norm(routed) * wr) * wf) * scalar.  `other` is a second status word
// (that of the routed branch) or null; sum is n floats of global scratch.
struct CombineArgs {
    const float *residual, *dense, *routed, *wd, *wr, *wf;
    float *sum, *out;
    int n;
    float eps, scalar;
    int *status;
    const int *other;
    // when expert_out is given, routed (writable then) is first filled with sum_k expert_out[k] * weights[k], k ascending
    const float *expert_out, *weights;
    int topk;
};

// n <= SQ_CHUNK: one load phase, everything else in registers and LDS
__global__ __launch_bounds__(THREADS) void combine_small_kernel(CombineArgs a) {
    __shared__ __attribute__((aligned(16))) float sq[2 * SQ_CHUNK + SQ_TAIL];
    __shared__ float shared[4];
    if (*a.status != 0) return;
    if (a.other && *a.other != 0) {
        if (threadIdx.x == 0) *a.status = -1;
        return;
    }
    unsigned bad = !(a.eps >= 0.0f) || nonfinite(a.eps) || nonfinite(a.scalar);
    float dr[2][SLOTS], res[SLOTS], wd[SLOTS], wr[SLOTS], wf[SLOTS];
#pragma unroll
    for (int k = 0; k < SLOTS; ++k) {
        const int i = (int)threadIdx.x + k * THREADS;
        const bool live = i < a.n;
        res[k] = live ? a.residual[i] : 0.0f;
        wd[k] = live ? a.wd[i] : 0.0f;
        wr[k] = live ? a.wr[i] : 0.0f;
        wf[k] = live ? a.wf[i] : 0.0f;
        dr[0][k] = live ? a.dense[i] : 0.0f;
        dr[1][k] = live && !a.expert_out ? a.routed[i] : 0.0f;
    }
    if (a.expert_out)
        for (int e = 0; e < a.topk; ++e) {
            const float w = a.weights[e];
#pragma unroll
            for (int k = 0; k < SLOTS; ++k) {
                const int i = (int)threadIdx.x + k * THREADS;
                if (i < a.n) {
                    const float term = a.expert_out[(size_t)e * a.n + i] * w;
                    dr[1][k] = dr[1][k] + term;
                }
            }
        }
#pragma unroll
    for (int k = 0; k < SLOTS; ++k)
        bad |= nonfinite(res[k]) | nonfinite(wd[k]) | nonfinite(wr[k]) | nonfinite(wf[k]) | nonfinite(dr[0][k]) |
               nonfinite(dr[1][k]);
    float ss[2];
    chains_from_registers<2>(dr, a.n, sq, shared, ss);
    const float inv_d = inverse_from_sum(ss[0], a.n, a.eps), inv_r = inverse_from_sum(ss[1], a.n, a.eps);
    bad |= nonfinite(inv_d) | nonfinite(inv_r);
    float sum[1][SLOTS];
#pragma unroll
    for (int k = 0; k < SLOTS; ++k) {
        const float d0 = dr[0][k] * inv_d, r0 = dr[1][k] * inv_r;
        const float d = d0 * wd[k], r = r0 * wr[k];
        sum[0][k] = d + r;
        bad |= nonfinite(d0) | nonfinite(r0) | nonfinite(d) | nonfinite(r) | nonfinite(sum[0][k]);
    }
    float ss_sum[1];
    chains_from_registers<1>(sum, a.n, sq, shared, ss_sum);
    const float inv_f = inverse_from_sum(ss_sum[0], a.n, a.eps);
    bad |= nonfinite(inv_f);
    float y[SLOTS];
#pragma unroll
    for (int k = 0; k < SLOTS; ++k) {
        const float f0 = sum[0][k] * inv_f;
        const float f = f0 * wf[k];
        y[k] = (res[k] + f) * a.scalar;
        bad |= nonfinite(f0) | nonfinite(f) | nonfinite(y[k]);
    }
    if (__syncthreads_or((int)bad)) {
        if (threadIdx.x == 0) *a.status = -1;
        return;
    }
#pragma unroll
    for (int k = 0; k < SLOTS; ++k) {
        const int i = (int)threadIdx.x + k * THREADS;
        if (i < a.n) a.out[i] = y[k];
    }
}

__global__ __launch_bounds__(THREADS) void combine_cell_kernel(CombineArgs a) {
    __shared__ __attribute__((aligned(16))) float sq[2 * SQ_CHUNK + SQ_TAIL];
    __shared__ float shared[4];
    if (*a.status != 0) return;
    if (a.other && *a.other != 0) {
        if (threadIdx.x == 0) *a.status = -1;
        return;
    }
    unsigned bad = !(a.eps >= 0.0f) || nonfinite(a.eps) || nonfinite(a.scalar);
    if (a.expert_out) {                                 // each thread later reads back only what it wrote here
        float *routed = const_cast<float *>(a.routed);
        for (int base = 0; base < a.n; base += SQ_CHUNK) {
            float sum[SLOTS];
#pragma unroll
            for (int k = 0; k < SLOTS; ++k) sum[k] = 0.0f;
            for (int e = 0; e < a.topk; ++e) {
                const float w = a.weights[e];
#pragma unroll
                for (int k = 0; k < SLOTS; ++k) {
                    const int i = base + (int)threadIdx.x + k * THREADS;
                    if (i < a.n) {
                        const float term = a.expert_out[(size_t)e * a.n + i] * w;
                        sum[k] = sum[k] + term;
                    }
                }
            }
#pragma unroll
            for (int k = 0; k < SLOTS; ++k) {
                const int i = base + (int)threadIdx.x + k * THREADS;
                if (i < a.n) routed[i] = sum[k];
            }
        }
    }
    const float *vec[2] = {a.dense, a.routed};
    float ss[2];
    serial_square_sums(vec, 2, a.n, sq, ss, shared, bad);
    const float inv_d = inverse_from_sum(ss[0], a.n, a.eps), inv_r = inverse_from_sum(ss[1], a.n, a.eps);
    bad |= nonfinite(inv_d) | nonfinite(inv_r);
    each_element(a.n, [&](int i) {
        const float wd = a.wd[i], wr = a.wr[i], res = a.residual[i], wf = a.wf[i];
        const float d0 = a.dense[i] * inv_d, r0 = a.routed[i] * inv_r;
        const float d = d0 * wd, r = r0 * wr;
        const float s = d + r;
        bad |= nonfinite(res) | nonfinite(wd) | nonfinite(wr) | nonfinite(wf) | nonfinite(d0) | nonfinite(r0) | nonfinite(d) | nonfinite(r) |
               nonfinite(s);
        a.sum[i] = s;
    });
    const float *vec2[1] = {a.sum};                     // a thread reads back the elements it wrote itself
    float ss_sum;
    serial_square_sums(vec2, 1, a.n, sq, &ss_sum, shared, bad);
    const float inv_f = inverse_from_sum(ss_sum, a.n, a.eps);
    bad |= nonfinite(inv_f);
    each_element(a.n, [&](int i) {
        const float f0 = a.sum[i] * inv_f;
        const float f = f0 * a.wf[i];
        const float y = (a.residual[i] + f) * a.scalar;
        bad |= nonfinite(f0) | nonfinite(f) | nonfinite(y);
    });
    if (__syncthreads_or((int)bad)) {
        if (threadIdx.x == 0) *a.status = -1;
        return;
    }
    each_element(a.n, [&](int i) {
        const float f = (a.sum[i] * inv_f) * a.wf[i];
        a.out[i] = (a.residual[i] + f) * a.scalar;
    });
}

constexpr int WIDE = 256;             // threads per workgroup of the grid-wide elementwise kernels

__global__ __launch_bounds__(WIDE) void finite_check_kernel(const float *x, size_t n, int *status) {
    unsigned bad = 0;
    for (size_t i = (size_t)blockIdx.x * WIDE + threadIdx.x; i < n; i += (size_t)gridDim.x * WIDE) bad |= nonfinite(x[i]);
    if (__syncthreads_or((int)bad) && threadIdx.x == 0) *status = -1;      // every writer stores the same value
}

__global__ __launch_bounds__(WIDE) void softcap_kernel(float *logits, size_t n, float cap, const int *status) {
    if (*status != 0) return;
    const size_t i = (size_t)blockIdx.x * WIDE + threadIdx.x;
    if (i < n) logits[i] = cap * det_tanhf(logits[i] / cap);
}

__global__ void merge_status_kernel(int *status, const int *other) {
    if (*other != 0) *status = -1;
}

bool launched() { return hipGetLastError() == hipSuccess; }

}  // namespace

int norm_cell_launch(int kind, const float *x, const float *weight, const float *residual, float *out, int n, float eps,
                     float root, int *status, hipStream_t stream) {
    if (!x || !out || !status || n < 1 || kind < 0 || kind > 2 || (kind != 0 && !weight) || (kind == 2 && !residual))
        return -1;
    NormArgs a = {x, weight, residual, out, n, kind, eps, root, status};
    norm_cell_kernel<<<dim3(1), dim3(THREADS), 0, stream>>>(a);
    return launched() ? 0 : -1;
}

int ffn_pre_launch(const float *residual, const float *w1, const float *w2, const float *router_scale, float *norm_a,
                   float *norm_b, float *router_in, int n, float eps, int *status, hipStream_t stream) {
    if (!residual || !w1 || !w2 || !router_scale || !norm_a || !norm_b || !router_in || !status || n < 1) return -1;
    PreArgs a = {residual, w1, w2, router_scale, norm_a, norm_b, router_in, n, eps, status};
    if (n <= SQ_CHUNK) ffn_pre_small_kernel<<<dim3(1), dim3(THREADS), 0, stream>>>(a);
    else ffn_pre_kernel<<<dim3(1), dim3(THREADS), 0, stream>>>(a);
    return launched() ? 0 : -1;
}

int combine_cell_launch(const float *residual, const float *dense, const float *routed, const float *wd, const float *wr,
                        const float *wf, float *sum_scratch, float *out, int n, float eps, float scalar, int *status,
                        const int *other_status, const float *expert_out, const float *weights, int topk,
                        hipStream_t stream) {
    if (!residual || !dense || !routed || !wd || !wr || !wf || !sum_scratch || !out || !status || n < 1 ||
        (expert_out && (!weights || topk < 1)))
        return -1;
    CombineArgs a = {residual, dense, routed, wd, wr, wf, sum_scratch, out, n, eps, scalar, status, other_status,
                     expert_out, weights, topk};
    if (n <= SQ_CHUNK) combine_small_kernel<<<dim3(1), dim3(THREADS), 0, stream>>>(a);
    else combine_cell_kernel<<<dim3(1), dim3(THREADS), 0, stream>>>(a);
    return launched() ? 0 : -1;
}

int softcap_cell_launch(float *logits, size_t n, float cap, int *status, hipStream_t stream) {
    if (!logits || !status || n < 1 || !(cap > 0.0f) || !(cap < __builtin_inff())) return -1;
    const size_t blocks = (n + WIDE - 1) / WIDE;
    finite_check_kernel<<<dim3((unsigned)(blocks < 1024 ? blocks : 1024)), dim3(WIDE), 0, stream>>>(logits, n, status);
    if (!launched()) return -1;
    softcap_kernel<<<dim3((unsigned)blocks), dim3(WIDE), 0, stream>>>(logits, n, cap, status);
    return launched() ? 0 : -1;
}

int merge_status_launch(int *status, const int *other, hipStream_t stream) {
    merge_status_kernel<<<dim3(1), dim3(1), 0, stream>>>(status, other);
    return launched() ? 0 : -1;
}

}  // namespace mi355
