// The activation side of the tolerance-class affine-Q4 kernels (q4_dot.hip, q4_dot16.hip): every 64-column group of
// an activation row becomes block fixed point, I_c = rint(x_c * 2^k) with |I_c| < 2^30, split into four signed 8-bit
// digit planes I = d0 + 2^8 d1 + 2^16 d2 + 2^24 d3, stored in LDS in the byte order in which the kernels unpack
// the weight codes; beside the digits the group's power of two 2^-k and its sum of activations (accumulated in
// double, rounded once).
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

// Called by every thread of the workgroup (THREADS of them, a multiple of 64).  load(t, column, xv) fetches the four
// activations of token t that start at `column`.  The caller places a barrier between this and the first read.
template <int T, int THREADS, class LoadX>
__device__ __forceinline__ void build_q4_image(int tid, int ngrp, int SG, uint8_t *zero_lds, uint8_t *img_lds, float *xm_lds,
                                               LoadX load) {
    for (int i = tid; i < ZERO_BYTES / 4; i += THREADS) ((uint32_t *)zero_lds)[i] = 0u;
    // one thread per four columns; the sixteen threads of a group are sixteen neighbouring lanes
    const int items = T * 2 * SG * 16;
    // items is a multiple of 64, so a wave is inside or outside a turn as a whole (the shuffles need that).  A thread
    // requests the activations of up to BATCH items before it works on the first: one memory latency per batch.
    constexpr int BATCH = 4;
    for (int first = tid; first < items; first += BATCH * THREADS) {
        float xs[BATCH][4];
#pragma unroll
        for (int k = 0; k < BATCH; ++k) {
            const int item = first + k * THREADS;
            xs[k][0] = xs[k][1] = xs[k][2] = xs[k][3] = 0.0f;
            if (item < items) {
                const int g = (item >> 4) % (2 * SG), t = (item >> 4) / (2 * SG);
                if (g < ngrp) load(t, (size_t)g * 64 + 4 * (item & 15), xs[k]);
            }
        }
#pragma unroll
        for (int k = 0; k < BATCH; ++k) {
            const int item = first + k * THREADS;
            if (item >= items) break;                  // wave-uniform
            const int q16 = item & 15;
            const int g = (item >> 4) % (2 * SG);      // slot of the group in the image = its index in the row
            const int t = (item >> 4) / (2 * SG);
            const bool valid = g < ngrp;               // slots past the row's end hold zero digits
            const float (&xv)[4] = xs[k];
            float gmax = __builtin_fmaxf(__builtin_fmaxf(__builtin_fabsf(xv[0]), __builtin_fabsf(xv[1])),
                                         __builtin_fmaxf(__builtin_fabsf(xv[2]), __builtin_fabsf(xv[3])));
            double gsum = ((double)xv[0] + (double)xv[1]) + ((double)xv[2] + (double)xv[3]);
            // a NaN does not survive the maximum, but the sum keeps it, and with it every output of the token
#pragma unroll
            for (int d = 1; d < 16; d <<= 1) {
                gmax = __builtin_fmaxf(gmax, __shfl_xor(gmax, d, 64));
                gsum = gsum + __shfl_xor(gsum, d, 64);
            }
            // gmax in [2^E, 2^(E+1)): digits of rint(x * 2^(29 - E)); tiny groups are pinned at E = -97
            int eb = (int)((__float_as_uint(gmax) >> 23) & 0xffu);
            eb = eb < 30 ? 30 : (eb > 254 ? 254 : eb);
            const float up = __uint_as_float((uint32_t)(283 - eb) << 23);      // 2^(29 - E)
            const float down = __uint_as_float((uint32_t)(eb - 29) << 23);     // 2^(E - 29)
            int d0[4], d1[4], d2[4], d3[4];
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                float scaled = xv[c] * up;
                scaled = __builtin_fminf(__builtin_fmaxf(scaled, -1073741824.0f), 1073741824.0f);   // non-finite input: any digits
                int I = __float2int_rn(scaled);
                d0[c] = (int)(int8_t)I; I = (I - d0[c]) >> 8;
                d1[c] = (int)(int8_t)I; I = (I - d1[c]) >> 8;
                d2[c] = (int)(int8_t)I; I = (I - d2[c]) >> 8;
                d3[c] = I;
            }
            // byte order inside a sixteen-column quarter = the order the code extraction yields:
            // columns 0 2 4 6 | 1 3 5 7 | 8 10 12 14 | 9 11 13 15
            const int j = q16 >> 2, c4 = (q16 & 3) * 4;
            const int pos = (c4 & 8) + ((c4 & 4) >> 1);
            uint8_t *slot = img_lds + ((size_t)(t * 2 * SG + g) * 16 + j * 4) * 16 + pos;
            const int *planes[4] = {d0, d1, d2, d3};
#pragma unroll
            for (int p = 0; p < 4; ++p) {
                const int *d = planes[p];
                *(uint16_t *)(slot + p * 16) = (uint16_t)((d[0] & 0xff) | ((d[2] & 0xff) << 8));
                *(uint16_t *)(slot + p * 16 + 4) = (uint16_t)((d[1] & 0xff) | ((d[3] & 0xff) << 8));
            }
            if (q16 == 0) {
                xm_lds[2 * (t * 2 * SG + g)] = valid ? down : 0.0f;
                xm_lds[2 * (t * 2 * SG + g) + 1] = valid ? (float)gsum : 0.0f;
            }
        }
    }
}

}  // namespace
}  // namespace mi355
