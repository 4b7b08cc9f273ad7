// The activation side of the tolerance-class affine-Q4 kernels (q4_dot.hip, q4_dot16.hip, moe_dot16.hip): every
// 64-column group of an activation row becomes block fixed point, I_c = rint(x_c * 2^k) with |I_c| <= 2^30, split
// into four signed 8-bit digit planes I = d0 + 2^8 d1 + 2^16 d2 + 2^24 d3, stored in LDS in the byte order in which
// the kernels unpack the weight codes; beside the digits the group's power of two 2^-k and the sum of the group's
// fixed-point image, sum_c I_c * 2^-k (an exact integer sum, rounded once).  The kernels therefore compute
// sum_c (q_c s + b) * xhat_c for the image xhat of x, which differs from x by at most 2^-30 of the group's largest
// magnitude per column.
//
// Image layout: [token][group slot 0 .. 2 * SG)[quarter of 16 columns][plane][16 bytes]; slots past the row's last
// group hold zero digits.  A 16-byte piece is the operand of one lane of the integer matrix instruction.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace mi355 {
namespace {

constexpr int ZERO_BYTES = 1024 + 256;       // what lanes without a digit plane read instead
constexpr int GROUP_IMAGE = 256;             // bytes of digits per group: 4 quarters x 4 planes x 16
constexpr int IMAGE_HELD = 2;                // items whose activations a thread may request ahead of the build

typedef float image_f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t image_u32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t image_u32x4 __attribute__((ext_vector_type(4)));

// All-reduce over the eight neighbouring lanes that share a group's octets, by data-parallel primitives inside the
// lanes' row (no LDS): lane ^ 1, lane ^ 2, then the mirror image of the half row.  Every exchange is evaluated once,
// by all lanes (a lane that skipped it would hand its neighbour nothing).
template <int CONTROL>
__device__ __forceinline__ uint32_t image_neighbour(uint32_t value) {
    return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)value, CONTROL, 0xf, 0xf, false);
}
__device__ __forceinline__ uint32_t image_max8(uint32_t value) {
    uint32_t other = image_neighbour<0xB1>(value);
    value = value > other ? value : other;
    other = image_neighbour<0x4E>(value);
    value = value > other ? value : other;
    other = image_neighbour<0x141>(value);
    return value > other ? value : other;
}
__device__ __forceinline__ int image_sum8(int value) {
    value += (int)image_neighbour<0xB1>((uint32_t)value);
    value += (int)image_neighbour<0x4E>((uint32_t)value);
    return value + (int)image_neighbour<0x141>((uint32_t)value);
}

// One item = eight consecutive columns of one group of one token (eight items, eight neighbouring lanes, per group).
// Items run densely over the real groups: item = (token * ngrp + group) * 8 + octet.
struct ImageItems {
    int ngrp, count;                         // groups per row; items in all
    __device__ __forceinline__ ImageItems(int tokens, int ngrp_) : ngrp(ngrp_), count(tokens * ngrp_ * 8) {}
};

// The digits, power of two and sum of one item whose eight activations are in xv; the eight lanes of a group call
// this together.  `live` is false for lanes past the last item (they compute on zeros and store nothing).
__device__ __forceinline__ void image_store_item(int item, bool live, const ImageItems &items, int SG, const float (&xv)[8],
                                                 uint8_t *img_lds, float *xm_lds) {
    const int octet = item & 7;
    const int slot_in_all = item >> 3;                         // token * ngrp + group
    const int t = slot_in_all / items.ngrp, g = slot_in_all - t * items.ngrp;
    // largest magnitude of the group as an integer maximum over the bit patterns: a NaN or an infinity wins it
    uint32_t top = 0u;
#pragma unroll
    for (int c = 0; c < 8; ++c) {
        const uint32_t mag = __float_as_uint(xv[c]) & 0x7fffffffu;
        top = top > mag ? top : mag;
    }
    top = image_max8(top);
    const bool finite = top < 0x7f800000u;
    // top in [2^E, 2^(E+1)): digits of rint(x * 2^(29 - E)); tiny groups are pinned at E = -97
    int eb = (int)(top >> 23);
    eb = eb < 30 ? 30 : (eb > 254 ? 254 : eb);
    const float up = __uint_as_float((uint32_t)(283 - eb) << 23);      // 2^(29 - E)
    const float down = __uint_as_float((uint32_t)(eb - 29) << 23);     // 2^(E - 29)
    // The four signed digits of I are the bytes of (I + 0x808080) ^ 0x808080: adding 128 to each of the three low
    // bytes carries exactly where a digit would be negative, and flipping the top bit turns byte b into b - 128.
    uint32_t k[8];
#pragma unroll
    for (int c = 0; c < 8; ++c) {
        const int I = (int)__builtin_rintf(xv[c] * up);                // a non-finite group: any digits
        k[c] = ((uint32_t)I + 0x00808080u) ^ 0x00808080u;
    }
    // byte order inside a sixteen-column quarter = the order the code extraction yields:
    // columns 0 2 4 6 | 1 3 5 7 | 8 10 12 14 | 9 11 13 15; plane p takes byte p of every column
    uint32_t even[4], odd[4];
    {
        const uint32_t a_lo = __builtin_amdgcn_perm(k[2], k[0], 0x05010400u), a_hi = __builtin_amdgcn_perm(k[2], k[0], 0x07030602u);
        const uint32_t b_lo = __builtin_amdgcn_perm(k[6], k[4], 0x05010400u), b_hi = __builtin_amdgcn_perm(k[6], k[4], 0x07030602u);
        even[0] = __builtin_amdgcn_perm(b_lo, a_lo, 0x05040100u); even[1] = __builtin_amdgcn_perm(b_lo, a_lo, 0x07060302u);
        even[2] = __builtin_amdgcn_perm(b_hi, a_hi, 0x05040100u); even[3] = __builtin_amdgcn_perm(b_hi, a_hi, 0x07060302u);
        const uint32_t c_lo = __builtin_amdgcn_perm(k[3], k[1], 0x05010400u), c_hi = __builtin_amdgcn_perm(k[3], k[1], 0x07030602u);
        const uint32_t d_lo = __builtin_amdgcn_perm(k[7], k[5], 0x05010400u), d_hi = __builtin_amdgcn_perm(k[7], k[5], 0x07030602u);
        odd[0] = __builtin_amdgcn_perm(d_lo, c_lo, 0x05040100u); odd[1] = __builtin_amdgcn_perm(d_lo, c_lo, 0x07060302u);
        odd[2] = __builtin_amdgcn_perm(d_hi, c_hi, 0x05040100u); odd[3] = __builtin_amdgcn_perm(d_hi, c_hi, 0x07060302u);
    }
    // sum of the group's image: plane sums by byte dot products, low and high pair of planes apart (each below 2^22)
    int plane_sum[4];
#pragma unroll
    for (int p = 0; p < 4; ++p)
        plane_sum[p] = __builtin_amdgcn_sdot4((int)odd[p], 0x01010101, __builtin_amdgcn_sdot4((int)even[p], 0x01010101, 0, false), false);
    int sum_lo = plane_sum[0] + plane_sum[1] * 256, sum_hi = plane_sum[2] + plane_sum[3] * 256;
    sum_lo = image_sum8(sum_lo);
    sum_hi = image_sum8(sum_hi);
    if (!live) return;
    uint8_t *piece = img_lds + ((size_t)(t * 2 * SG + g) * 16 + (octet >> 1) * 4) * 16 + (octet & 1) * 8;
#pragma unroll
    for (int p = 0; p < 4; ++p) *(image_u32x2 *)(piece + p * 16) = image_u32x2{even[p], odd[p]};
    if (octet == 0) {
        const float total = __builtin_fmaf((float)sum_hi, 65536.0f, (float)sum_lo);       // the integer sum, rounded once
        // a non-finite activation poisons every output of its token through the bias term
        xm_lds[2 * (t * 2 * SG + g)] = down;
        xm_lds[2 * (t * 2 * SG + g) + 1] = finite ? total * down : __uint_as_float(0x7fc00000u);
    }
}

// Turns of the workgroup over the items.  request() asks for the activations of the thread's first IMAGE_HELD items
// and may be called long before build(): whatever the caller issues in between (weight loads) then queues behind
// them, not in front.  load(t, column, xv) fetches the eight activations of token t that start at `column`.
template <int THREADS>
struct Q4ImageBuilder {
    float held[IMAGE_HELD][8];
    image_f32x4 early[IMAGE_HELD][2];

    template <class LoadX>
    __device__ __forceinline__ void request(int tid, const ImageItems &items, LoadX load) {
#pragma unroll
        for (int k = 0; k < IMAGE_HELD; ++k) {
            const int item = tid + k * THREADS;
#pragma unroll
            for (int c = 0; c < 8; ++c) held[k][c] = 0.0f;
            if (item < items.count) {
                const int slot = item >> 3, t = slot / items.ngrp, g = slot - t * items.ngrp;
                load(t, (size_t)g * 64 + 8 * (item & 7), held[k]);
            }
        }
    }

    // The same request with loads the compiler neither moves nor waits for (32-byte aligned rows of activations):
    // the caller goes on with other work and calls settle() before build().
    template <class RowOf>
    __device__ __forceinline__ void request_early(int tid, const ImageItems &items, RowOf row_of) {
#pragma unroll
        for (int k = 0; k < IMAGE_HELD; ++k) {
            if (k * THREADS >= items.count) break;               // uniform
            int item = tid + k * THREADS;
            item = item < items.count ? item : items.count - 1;  // lanes past the end repeat the last item (never stored)
            const int slot = item >> 3, t = slot / items.ngrp, g = slot - t * items.ngrp;
            const float *src = row_of(t) + (size_t)g * 64 + 8 * (item & 7);
            // the values stay in the registers the loads write until settle(): a copy made now would read them
            // before the data has arrived
            asm volatile("global_load_dwordx4 %0, %2, off\n\tglobal_load_dwordx4 %1, %2, off offset:16"
                         : "=&v"(early[k][0]), "=&v"(early[k][1]) : "v"(src) : "memory");
        }
    }
    // Waits for everything the wave has in flight and ties the requested values to that wait (`after` is any value
    // the caller computed from loads issued after request_early: the wait then cannot move in front of them).
    __device__ __forceinline__ void settle(int after, const ImageItems &items) {
#pragma unroll
        for (int k = 0; k < IMAGE_HELD; ++k) {
            if (k * THREADS >= items.count) break;               // uniform
            asm volatile("s_waitcnt vmcnt(0)" : "+v"(early[k][0]), "+v"(early[k][1]) : "s"(after) : "memory");
            held[k][0] = early[k][0].x; held[k][1] = early[k][0].y; held[k][2] = early[k][0].z; held[k][3] = early[k][0].w;
            held[k][4] = early[k][1].x; held[k][5] = early[k][1].y; held[k][6] = early[k][1].z; held[k][7] = early[k][1].w;
        }
    }

    // Called by every thread of the workgroup.  The caller places a barrier between this and the first read.
    template <class LoadX>
    __device__ __forceinline__ void build(int tid, const ImageItems &items, int SG, uint8_t *zero_lds, uint8_t *img_lds,
                                          float *xm_lds, LoadX load) {
        for (int i = tid; i < ZERO_BYTES / 4; i += THREADS) ((uint32_t *)zero_lds)[i] = 0u;
        // slots past the row's last group: zero digits, zero factors
        const int tokens = items.count / (items.ngrp * 8), spare = 2 * SG - items.ngrp;
        for (int i = tid; i < tokens * spare * 16; i += THREADS) {
            const int t = i / (spare * 16), rest = i - t * (spare * 16);
            *(image_u32x4 *)(img_lds + ((size_t)(t * 2 * SG + items.ngrp) * 16 + rest) * 16) = image_u32x4{0u, 0u, 0u, 0u};
        }
        for (int i = tid; i < tokens * spare; i += THREADS) {
            const int t = i / spare, g = items.ngrp + (i - t * spare);
            xm_lds[2 * (t * 2 * SG + g)] = 0.0f;
            xm_lds[2 * (t * 2 * SG + g) + 1] = 0.0f;
        }
#pragma unroll
        for (int k = 0; k < IMAGE_HELD; ++k) {
            const int item = tid + k * THREADS;
            if (k * THREADS >= items.count) break;               // uniform
            image_store_item(item < items.count ? item : items.count - 1, item < items.count, items, SG, held[k], img_lds, xm_lds);
        }
        // wide rows or several tokens: further turns, IMAGE_HELD requests at a time
        for (int base = IMAGE_HELD * THREADS; base < items.count; base += IMAGE_HELD * THREADS) {
            float xs[IMAGE_HELD][8];
#pragma unroll
            for (int k = 0; k < IMAGE_HELD; ++k) {
                const int item = base + tid + k * THREADS;
#pragma unroll
                for (int c = 0; c < 8; ++c) xs[k][c] = 0.0f;
                if (item < items.count) {
                    const int slot = item >> 3, t = slot / items.ngrp, g = slot - t * items.ngrp;
                    load(t, (size_t)g * 64 + 8 * (item & 7), xs[k]);
                }
            }
#pragma unroll
            for (int k = 0; k < IMAGE_HELD; ++k) {
                const int item = base + tid + k * THREADS;
                if (base + k * THREADS >= items.count) break;    // uniform
                image_store_item(item < items.count ? item : items.count - 1, item < items.count, items, SG, xs[k], img_lds, xm_lds);
            }
        }
    }
};

// request() and build() back to back, for T tokens (T = 0: `tokens` of them, known at run time).
template <int T, int THREADS, class LoadX>
__device__ __forceinline__ void build_q4_image(int tid, int ngrp, int SG, uint8_t *zero_lds, uint8_t *img_lds, float *xm_lds,
                                               int tokens, LoadX load) {
    const ImageItems items(T > 0 ? T : tokens, ngrp);
    Q4ImageBuilder<THREADS> builder;
    builder.request(tid, items, load);
    builder.build(tid, items, SG, zero_lds, img_lds, xm_lds, load);
}

// A window of the row, for kernels that hold only part of a wide row's image at a time.  The slots are
// [token][strip 0 | strip 1][SGw]; they take the groups first .. first + groups_here of each strip (strip 1 starts at
// group SG of the row).  Slots whose group lies past the window's or the row's end hold zero digits.  The zero region
// is not written here.  request() fetches the activations of the thread's first items and may be called well before
// build() (before the walk over the window in front, so that the walk hides the fetch).
template <int T, int THREADS>
struct Q4WindowBuilder {
    static constexpr int BATCH = 4;
    float xs[BATCH][8];
    int ngrp, SG, first, groups_here, SGw;

    __device__ __forceinline__ void window(int ngrp_, int SG_, int first_, int groups_here_, int SGw_) {
        ngrp = ngrp_; SG = SG_; first = first_; groups_here = groups_here_; SGw = SGw_;
    }
    template <class LoadX>
    __device__ __forceinline__ void fetch(int base, int tid, LoadX load) {
        const int count = T * 2 * SGw * 8;
#pragma unroll
        for (int k = 0; k < BATCH; ++k) {
            const int item = base + tid + k * THREADS;
#pragma unroll
            for (int c = 0; c < 8; ++c) xs[k][c] = 0.0f;
            if (item < count) {
                const int slot = item >> 3, t = slot / (2 * SGw), w = slot - t * (2 * SGw);
                const int strip = w >= SGw ? 1 : 0, gw = w - strip * SGw, g = strip * SG + first + gw;
                if (gw < groups_here && g < ngrp) load(t, (size_t)g * 64 + 8 * (item & 7), xs[k]);
            }
        }
    }
    template <class LoadX>
    __device__ __forceinline__ void request(int tid, LoadX load) { fetch(0, tid, load); }

    template <class LoadX>
    __device__ __forceinline__ void build(int tid, uint8_t *img_lds, float *xm_lds, LoadX load) {
        const ImageItems slots(T, 2 * SGw);
        for (int base = 0; base < slots.count; base += BATCH * THREADS) {
            if (base > 0) fetch(base, tid, load);
#pragma unroll
            for (int k = 0; k < BATCH; ++k) {
                const int item = base + tid + k * THREADS;
                if (base + k * THREADS >= slots.count) break;        // uniform
                image_store_item(item < slots.count ? item : slots.count - 1, item < slots.count, slots, SGw, xs[k], img_lds, xm_lds);
            }
        }
    }
};

}  // namespace
}  // namespace mi355
