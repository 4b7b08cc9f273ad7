/* salt_gpu_mi355.h -- C ABI of libsalt_gpu_mi355.so, the MI355X (gfx950)
 * backend for SALT's quantized decode path.
 *
 * Two groups of entry points:
 *
 *  1. The engine's physical-backend ABI for this path.  These carry the names
 *     and signatures of the reference's include/salt/gpu.h so that linking this
 *     library in place of the reference's gpu_hip.o / gpu_stub.o needs no
 *     engine change; each declaration cites the reference lines it replaces.
 *     All pointers are host pointers owned by the caller; 0 = done, -1 =
 *     unavailable or failed (reference gpu.h:23-25).  They are declared in
 *     salt_gpu_mi355_engine.h, which this header includes.
 *
 *  2. Device-resident entry points (salt_mi355_*): the same operations on
 *     buffers that already live in HBM, launched on a caller-supplied HIP
 *     stream.  The engine-facing calls are thin host wrappers around these.
 *     They have no counterpart in the reference ABI, whose every call moves
 *     activations across the host boundary; harnesses that keep data on the
 *     device (the benchmark, the parity tests, a future whole-layer program)
 *     call them directly.
 *
 * Plain C, no HIP or torch types: a stream is passed as void* (hipStream_t,
 * NULL = the null stream) and device memory as void* / typed pointers.
 * The library is not thread-safe; like the reference backends it expects one
 * owner thread (reference gpu_hip.cpp keeps global state without locks).
 */
#ifndef SALT_GPU_MI355_H
#define SALT_GPU_MI355_H

#include <stddef.h>
#include <stdint.h>

#include "salt_gpu_mi355_engine.h"

#ifdef __cplusplus
extern "C" {
#endif

/* ---- lifecycle and diagnostics ---------------------------------------- */

/* Selects device 0, creates the library stream, and checks on the device that
 * the fp8 and fp4 converters decode the way the kernels assume.  Idempotent.
 * salt_gpu_init (reference gpu.h:26) calls this. */
int salt_mi355_init(void);
int salt_mi355_shutdown(void);
/* Last failure recorded by any entry point, for logs; never NULL. */
const char *salt_mi355_last_error(void);
/* Raw decode tables measured at init: fp8[b] is what v_cvt_pk_f32_fp8 returns
 * for byte b; fp4[2*b], fp4[2*b+1] what v_cvt_scalef32_pk_f32_fp4 (scale 1)
 * returns for the low and high nibble of byte b.  Host arrays of 256 / 512. */
int salt_mi355_converter_tables(float *fp8, float *fp4);

/* ---- device memory and timing helpers for host harnesses --------------- */

void *salt_mi355_dev_alloc(size_t nbytes);
int salt_mi355_dev_free(void *device_ptr);
int salt_mi355_dev_upload(void *device_dst, const void *host_src, size_t nbytes);
int salt_mi355_dev_download(void *host_dst, const void *device_src, size_t nbytes);
int salt_mi355_dev_fill(void *device_dst, int byte_value, size_t nbytes);
/* The library's own stream (default priority), as a hipStream_t. */
void *salt_mi355_stream(void);
int salt_mi355_stream_sync(void *stream);
void *salt_mi355_event_create(void);
int salt_mi355_event_destroy(void *event);
int salt_mi355_event_record(void *event, void *stream);
/* Waits for `stop`, then returns the milliseconds between the two events. */
int salt_mi355_event_elapsed_ms(void *start, void *stop, float *ms);

/* ---- affine Q4 ("mlx4") matvec, device-resident ------------------------
 * Layout as the reference's salt_q4_matvec (kernels.h:117-130): u32 words of
 * eight nibbles, low nibble first, flat element index r*C + c; one bf16 scale
 * and one bf16 bias per 64 flat elements (biases may be NULL: bias 0).
 * ys[t*R + r] is bit-identical to the reference CPU row (kernels.c:220-250)
 * against xs[t*C ..].  B >= 1 tokens; weights are streamed once per group of
 * four tokens.  chains_per_lane: 0 = choose, or 8 / 4 / 2 (tuning knob). */
int salt_mi355_q4_matvec_dev(const void *vals, const void *scales, const void *biases,
                             int R, int C, int B, const float *xs, float *ys,
                             int chains_per_lane, void *stream);

/* Many matrices in one launch (the shape of reference salt_gpu_q4_batch,
 * gpu.h:83): job j multiplies its own R_j x C matrix with its own tokens.
 * `jobs` is a HOST array; the library copies it to the device on `stream`. */
typedef struct SaltMi355Q4Job {
    const void *vals;
    const void *scales;
    const void *biases;      /* may be NULL */
    const float *xs;         /* device, [tokens][C] */
    float *ys;               /* device, [tokens][rows] */
    int rows;
} SaltMi355Q4Job;
int salt_mi355_q4_jobs_dev(const SaltMi355Q4Job *jobs, int njobs, int C, int tokens,
                           int chains_per_lane, void *stream);

#ifdef __cplusplus
}
#endif

#endif /* SALT_GPU_MI355_H */
