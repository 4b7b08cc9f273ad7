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

constexpr int THREADS = 256;
constexpr int SQ_CHUNK = 4096;          // squares staged per pass of the serial adder

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

__device__ __forceinline__ bool finite(float v) { return (__float_as_uint(v) & 0x7f800000u) != 0x7f800000u; }

// Serial sums of squares of `vectors` (1..4) vectors of n floats: vector v is x[v].  Returns the sums in ss[] on
// every thread.  bad is set when an element is not finite.  sq is LDS scratch of vectors * SQ_CHUNK floats.
__device__ void serial_square_sums(const float *const *x, int vectors, int n, float *sq, float *ss_out, float *shared,
                                   bool &bad) {
    const int tid = threadIdx.x;
    float acc = 0.0f;                                   // lane v of wave 0 owns vector v
    for (int base = 0; base < n; base += SQ_CHUNK) {
        const int count = n - base < SQ_CHUNK ? n - base : SQ_CHUNK;
        for (int v = 0; v < vectors; ++v)
            for (int i = tid; i < count; i += THREADS) {
                const float value = x[v][base + i];
                bad = bad || !finite(value);
                sq[v * SQ_CHUNK + i] = value * value;
            }
        __syncthreads();
        if (tid < vectors) {
            const float *mine = sq + tid * SQ_CHUNK;
            int i = 0;
            for (; i + 16 <= count; i += 16) {
                float4 p[4];
#pragma unroll
                for (int k = 0; k < 4; ++k) p[k] = *(const float4 *)&mine[i + 4 * k];
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    acc = acc + p[k].x;
                    acc = acc + p[k].y;
                    acc = acc + p[k].z;
                    acc = acc + p[k].w;
                }
            }
            for (; i < count; ++i) acc = acc + mine[i];
        }
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
    __shared__ __attribute__((aligned(16))) float sq[SQ_CHUNK];
    __shared__ float shared[4];
    if (*a.status != 0) return;
    bool bad = !(a.eps >= 0.0f) || !finite(a.eps);
    const float *vec[1] = {a.x};
    float ss;
    serial_square_sums(vec, 1, a.n, sq, &ss, shared, bad);
    const float inv = inverse_from_sum(ss, a.n, a.eps);
    bad = bad || !finite(inv);
    float root = a.root;
    if (a.kind == 1 && !(root > 0.0f)) root = 1.0f / det_sqrtf((float)a.n);
    for (int i = threadIdx.x; i < a.n; i += THREADS) {
        float y = a.x[i] * inv;
        if (a.weight) { bad = bad || !finite(a.weight[i]); y = y * a.weight[i]; }
        if (a.kind == 1) y = y * root;
        bad = bad || !finite(y);
        if (a.kind == 2) {
            bad = bad || !finite(a.residual[i]);
            bad = bad || !finite(a.residual[i] + y);
        }
    }
    if (__syncthreads_or(bad)) {
        if (threadIdx.x == 0) *a.status = -1;
        return;
    }
    for (int i = threadIdx.x; i < a.n; i += THREADS) {
        float y = a.x[i] * inv;
        if (a.weight) y = y * a.weight[i];
        if (a.kind == 1) y = y * root;
        if (a.kind == 2) y = a.residual[i] + y;
        a.out[i] = y;
    }
}

// One pass over the residual for the three vectors a feed-forward block derives from it:
// norm_a = (r * inv) * w1, router_in = ((r * inv) * scale) * root, norm_b = (r * inv) * w2.
struct PreArgs {
    const float *residual, *w1, *w2, *router_scale;
    float *norm_a, *norm_b, *router_in;
    int n;
    float eps;
    int *status;
};

__global__ __launch_bounds__(THREADS) void ffn_pre_kernel(PreArgs a) {
    __shared__ __attribute__((aligned(16))) float sq[SQ_CHUNK];
    __shared__ float shared[4];
    if (*a.status != 0) return;
    bool bad = !(a.eps >= 0.0f) || !finite(a.eps);
    const float *vec[1] = {a.residual};
    float ss;
    serial_square_sums(vec, 1, a.n, sq, &ss, shared, bad);
    const float inv = inverse_from_sum(ss, a.n, a.eps);
    bad = bad || !finite(inv);
    const float root = 1.0f / det_sqrtf((float)a.n);
    for (int i = threadIdx.x; i < a.n; i += THREADS) {
        const float y = a.residual[i] * inv;
        bad = bad || !finite(a.w1[i]) || !finite(a.w2[i]) || !finite(a.router_scale[i]);
        bad = bad || !finite(y) || !finite(y * a.w1[i]) || !finite(y * a.w2[i]) || !finite((y * a.router_scale[i]) * root);
    }
    if (__syncthreads_or(bad)) {
        if (threadIdx.x == 0) *a.status = -1;
        return;
    }
    for (int i = threadIdx.x; i < a.n; i += THREADS) {
        const float y = a.residual[i] * inv;
        a.norm_a[i] = y * a.w1[i];
        a.norm_b[i] = y * a.w2[i];
        a.router_in[i] = (y * a.router_scale[i]) * root;
    }
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
};

__global__ __launch_bounds__(THREADS) void combine_cell_kernel(CombineArgs a) {
    __shared__ __attribute__((aligned(16))) float sq[2 * SQ_CHUNK];
    __shared__ float shared[4];
    if (*a.status != 0) return;
    if (a.other && *a.other != 0) {
        if (threadIdx.x == 0) *a.status = -1;
        return;
    }
    bool bad = !(a.eps >= 0.0f) || !finite(a.eps) || !finite(a.scalar);
    const float *vec[2] = {a.dense, a.routed};
    float ss[2];
    serial_square_sums(vec, 2, a.n, sq, ss, shared, bad);
    const float inv_d = inverse_from_sum(ss[0], a.n, a.eps), inv_r = inverse_from_sum(ss[1], a.n, a.eps);
    bad = bad || !finite(inv_d) || !finite(inv_r);
    for (int i = threadIdx.x; i < a.n; i += THREADS) {
        const float d = (a.dense[i] * inv_d) * a.wd[i], r = (a.routed[i] * inv_r) * a.wr[i];
        const float s = d + r;
        bad = bad || !finite(a.residual[i]) || !finite(a.wd[i]) || !finite(a.wr[i]) || !finite(a.wf[i]);
        bad = bad || !finite(a.dense[i] * inv_d) || !finite(a.routed[i] * inv_r) || !finite(d) || !finite(r) || !finite(s);
        a.sum[i] = s;
    }
    __syncthreads();                                    // a.sum is read back by other threads below
    const float *vec2[1] = {a.sum};
    float ss_sum;
    serial_square_sums(vec2, 1, a.n, sq, &ss_sum, shared, bad);
    const float inv_f = inverse_from_sum(ss_sum, a.n, a.eps);
    bad = bad || !finite(inv_f);
    for (int i = threadIdx.x; i < a.n; i += THREADS) {
        const float f = (a.sum[i] * inv_f) * a.wf[i];
        const float y = (a.residual[i] + f) * a.scalar;
        bad = bad || !finite(a.sum[i] * inv_f) || !finite(f) || !finite(y);
    }
    if (__syncthreads_or(bad)) {
        if (threadIdx.x == 0) *a.status = -1;
        return;
    }
    for (int i = threadIdx.x; i < a.n; i += THREADS) {
        const float f = (a.sum[i] * inv_f) * a.wf[i];
        a.out[i] = (a.residual[i] + f) * a.scalar;
    }
}

__global__ __launch_bounds__(THREADS) void finite_check_kernel(const float *x, size_t n, int *status) {
    bool bad = false;
    for (size_t i = (size_t)blockIdx.x * THREADS + threadIdx.x; i < n; i += (size_t)gridDim.x * THREADS)
        bad = bad || !finite(x[i]);
    if (__syncthreads_or(bad) && threadIdx.x == 0) *status = -1;      // every writer stores the same value
}

__global__ __launch_bounds__(THREADS) void softcap_kernel(float *logits, size_t n, float cap, const int *status) {
    if (*status != 0) return;
    const size_t i = (size_t)blockIdx.x * THREADS + threadIdx.x;
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
    ffn_pre_kernel<<<dim3(1), dim3(THREADS), 0, stream>>>(a);
    return launched() ? 0 : -1;
}

int combine_cell_launch(const float *residual, const float *dense, const float *routed, const float *wd, const float *wr,
                        const float *wf, float *sum_scratch, float *out, int n, float eps, float scalar, int *status,
                        const int *other_status, hipStream_t stream) {
    if (!residual || !dense || !routed || !wd || !wr || !wf || !sum_scratch || !out || !status || n < 1) return -1;
    CombineArgs a = {residual, dense, routed, wd, wr, wf, sum_scratch, out, n, eps, scalar, status, other_status};
    combine_cell_kernel<<<dim3(1), dim3(THREADS), 0, stream>>>(a);
    return launched() ? 0 : -1;
}

int softcap_cell_launch(float *logits, size_t n, float cap, int *status, hipStream_t stream) {
    if (!logits || !status || n < 1 || !(cap > 0.0f) || !(cap < __builtin_inff())) return -1;
    const size_t blocks = (n + THREADS - 1) / THREADS;
    finite_check_kernel<<<dim3((unsigned)(blocks < 1024 ? blocks : 1024)), dim3(THREADS), 0, stream>>>(logits, n, status);
    if (!launched()) return -1;
    softcap_kernel<<<dim3((unsigned)blocks), dim3(THREADS), 0, stream>>>(logits, n, cap, status);
    return launched() ? 0 : -1;
}

int merge_status_launch(int *status, const int *other, hipStream_t stream) {
    merge_status_kernel<<<dim3(1), dim3(1), 0, stream>>>(status, other);
    return launched() ? 0 : -1;
}

}  // namespace mi355
