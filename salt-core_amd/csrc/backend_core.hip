// Library state, diagnostics, device helpers and the device-resident Q4 entry
// points of libsalt_gpu_mi355.so.
#include "backend_state.h"

#include <math.h>
#include <stdarg.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

namespace mi355 {

State g_state;

void set_error(const char *format, ...) {
    va_list args;
    va_start(args, format);
    vsnprintf(g_state.last_error, sizeof g_state.last_error, format, args);
    va_end(args);
    if (getenv("SALT_GPU_DIAG")) fprintf(stderr, "salt-mi355: %s\n", g_state.last_error);
}

void note_kernel(const char *format, ...) {
    va_list args;
    va_start(args, format);
    vsnprintf(g_state.last_kernel, sizeof g_state.last_kernel, format, args);
    va_end(args);
}

int hip_ok(hipError_t status, const char *what) {
    if (status == hipSuccess) return 0;
    set_error("%s: %s", what, hipGetErrorString(status));
    return -1;
}

namespace {

// What the kernels assume of the two converters, checked once on the device:
// a byte 0..15 through the fp8 converter is an exact multiple k * v(1) of the
// value it gives byte 1 (a power of two), and every fp4 code decodes to the
// E2M1 magnitude with its sign.
int verify_converters() {
    float *device = nullptr;
    if (hip_ok(hipMalloc((void **)&device, (256 + 512) * sizeof(float)), "hipMalloc probe") != 0) return -1;
    int rc = probe_converters_launch(device, device + 256, g_state.stream);
    if (rc == 0) rc = hip_ok(hipStreamSynchronize(g_state.stream), "converter probe");
    if (rc == 0)
        rc = hip_ok(hipMemcpy(g_state.fp8_table, device, 256 * sizeof(float), hipMemcpyDeviceToHost), "probe copy");
    if (rc == 0)
        rc = hip_ok(hipMemcpy(g_state.fp4_table, device + 256, 512 * sizeof(float), hipMemcpyDeviceToHost),
                    "probe copy");
    (void)hipFree(device);
    if (rc != 0) return -1;
    const float unit = g_state.fp8_table[1];
    int exponent = 0;
    if (!(unit > 0.0f) || frexpf(unit, &exponent) != 0.5f) {
        set_error("fp8 converter: byte 1 decodes to %g, not a power of two", (double)unit);
        return -1;
    }
    for (int k = 0; k < 16; ++k)
        if (g_state.fp8_table[k] != (float)k * unit) {
            set_error("fp8 converter: byte %d decodes to %g, expected %g", k, (double)g_state.fp8_table[k],
                      (double)((float)k * unit));
            return -1;
        }
    g_state.code_scale = 1.0f / unit;
    // NVFP4 block scales are OCP E4M3FN (bias 7, 0x7f / 0xff = NaN, no infinities)
    int ocp = 1;
    for (int code = 0; code < 256 && ocp; ++code) {
        const int e = (code >> 3) & 15, m = code & 7;
        const float got = g_state.fp8_table[code];
        if (e == 15 && m == 7) { ocp = got != got; continue; }
        float want = e == 0 ? (float)m * 0.001953125f : (1.0f + (float)m * 0.125f) * ldexpf(1.0f, e - 7);
        if (code & 0x80) want = -want;
        ocp = got == want;
    }
    g_state.fp8_is_ocp = ocp;
    static const float magnitude[8] = {0.0f, 0.5f, 1.0f, 1.5f, 2.0f, 3.0f, 4.0f, 6.0f};
    for (int byte = 0; byte < 256; ++byte)
        for (int half = 0; half < 2; ++half) {
            const int code = half ? byte >> 4 : byte & 15;
            const float want = (code & 8) ? -magnitude[code & 7] : magnitude[code & 7];
            if (g_state.fp4_table[2 * byte + half] != want) {   // -0 == +0 here on purpose
                set_error("fp4 converter: code %d decodes to %g, expected %g", code,
                          (double)g_state.fp4_table[2 * byte + half], (double)want);
                return -1;
            }
        }
    return 0;
}

}  // namespace

State::TableSlot *table_acquire(const void *host_table, size_t nbytes, hipStream_t stream) {
    State &s = g_state;
    // Not under stream capture: the ring waits on events and rewrites pinned memory between calls, and a captured
    // upload would not have run when the next call compares bytes.  Launches whose jobs travel in the kernel
    // arguments (up to Q4_INLINE_JOBS) need no table and can be captured.
    hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(stream, &capture) != hipSuccess) { (void)hipGetLastError(); capture = hipStreamCaptureStatusNone; }
    if (capture != hipStreamCaptureStatusNone) {
        set_error("a launch of more than %d jobs uploads a job table and cannot be captured into a graph", Q4_INLINE_JOBS);
        return nullptr;
    }
    // A decode loop sends the same tables token after token: a slot that already holds these bytes, uploaded on this
    // stream, is used again without a copy (stream order puts the earlier upload before the new reader).
    for (State::TableSlot &held : s.tables)
        if (held.device && held.valid_bytes == nbytes && held.stream == stream && memcmp(held.pinned, host_table, nbytes) == 0)
            return &held;
    State::TableSlot *slot = &s.tables[s.next_table];
    s.next_table = (s.next_table + 1) % State::kTableSlots;
    if (slot->busy) {
        if (hip_ok(hipEventSynchronize(slot->done), "job table slot reuse") != 0) return nullptr;
        slot->busy = 0;
    }
    if (nbytes > slot->capacity) {
        if (slot->device) { (void)hipFree(slot->device); (void)hipHostFree(slot->pinned); }
        slot->device = slot->pinned = nullptr;
        slot->capacity = 0;
        size_t capacity = 16 * 1024;
        while (capacity < nbytes) capacity *= 2;
        if (hip_ok(hipMalloc(&slot->device, capacity), "hipMalloc job table") != 0 ||
            hip_ok(hipHostMalloc(&slot->pinned, capacity, hipHostMallocDefault), "hipHostMalloc job table") != 0)
            return nullptr;
        slot->capacity = capacity;
    }
    if (!slot->done && hip_ok(hipEventCreateWithFlags(&slot->done, hipEventDisableTiming), "hipEventCreate") != 0)
        return nullptr;
    slot->valid_bytes = 0;
    memcpy(slot->pinned, host_table, nbytes);
    if (hip_ok(hipMemcpyAsync(slot->device, slot->pinned, nbytes, hipMemcpyHostToDevice, stream),
               "job table upload") != 0)
        return nullptr;
    slot->valid_bytes = nbytes;
    slot->stream = stream;
    return slot;
}

void table_release(State::TableSlot *slot, hipStream_t stream) {
    if (slot && hip_ok(hipEventRecord(slot->done, stream), "job table event") == 0) slot->busy = 1;
}

}  // namespace mi355

using namespace mi355;

extern "C" {

int salt_mi355_init(void) {
    State &s = g_state;
    if (s.ready) return 0;
    int count = 0;
    if (hip_ok(hipGetDeviceCount(&count), "hipGetDeviceCount") != 0 || count < 1) {
        if (count < 1) set_error("no HIP device");
        return -1;
    }
    hipDeviceProp_t prop;
    // The owner thread waits for every call's completion: spinning on it answers microseconds sooner than blocking.
    (void)hipSetDeviceFlags(hipDeviceScheduleSpin);
    (void)hipGetLastError();                     // refused when the process has already touched the device: harmless
    if (hip_ok(hipSetDevice(0), "hipSetDevice") != 0 ||
        hip_ok(hipGetDeviceProperties(&prop, 0), "hipGetDeviceProperties") != 0)
        return -1;
    if (strncmp(prop.gcnArchName, "gfx950", 6) != 0) {
        set_error("device is %s; this library carries gfx950 code only", prop.gcnArchName);
        return -1;
    }
    s.compute_units = prop.multiProcessorCount;
    if (hip_ok(hipStreamCreateWithFlags(&s.stream, hipStreamNonBlocking), "hipStreamCreate") != 0) return -1;
    if (hip_ok(hipStreamCreateWithFlags(&s.side, hipStreamNonBlocking), "hipStreamCreate side") != 0 ||
        hip_ok(hipEventCreateWithFlags(&s.fork, hipEventDisableTiming | hipEventDisableSystemFence), "hipEventCreate fork") != 0 ||
        hip_ok(hipEventCreateWithFlags(&s.join, hipEventDisableTiming | hipEventDisableSystemFence), "hipEventCreate join") != 0 ||
        verify_converters() != 0) {
        (void)hipStreamDestroy(s.stream);
        if (s.side) (void)hipStreamDestroy(s.side);
        if (s.fork) (void)hipEventDestroy(s.fork);
        if (s.join) (void)hipEventDestroy(s.join);
        s.stream = s.side = nullptr;
        s.fork = s.join = nullptr;
        return -1;
    }
    if (moe_static_scratch_prepare() != 0) return -1;
    s.ready = 1;
    if (getenv("SALT_GPU_DIAG"))
        fprintf(stderr, "salt-mi355: ready on %s, %d CUs, fp8 code scale %g\n", prop.gcnArchName,
                s.compute_units, (double)s.code_scale);
    return 0;
}

int salt_mi355_shutdown(void) {
    State &s = g_state;
    if (!s.ready) return 0;
    int failed = hip_ok(hipDeviceSynchronize(), "hipDeviceSynchronize at shutdown");
    for (State::TableSlot &slot : s.tables) {
        if (slot.device) { (void)hipFree(slot.device); (void)hipHostFree(slot.pinned); }
        if (slot.done) (void)hipEventDestroy(slot.done);
    }
    if (s.stream) failed |= hip_ok(hipStreamDestroy(s.stream), "hipStreamDestroy");
    if (s.side) failed |= hip_ok(hipStreamDestroy(s.side), "hipStreamDestroy side");
    if (s.fork) (void)hipEventDestroy(s.fork);
    if (s.join) (void)hipEventDestroy(s.join);
    char keep[sizeof s.last_error];
    memcpy(keep, s.last_error, sizeof keep);
    s = State();
    memcpy(s.last_error, keep, sizeof keep);
    return failed ? -1 : 0;
}

const char *salt_mi355_last_error(void) { return g_state.last_error; }
const char *salt_mi355_last_kernel(void) { return g_state.last_kernel; }

int salt_mi355_converter_tables(float *fp8, float *fp4) {
    if (!g_state.ready || !fp8 || !fp4) return -1;
    memcpy(fp8, g_state.fp8_table, sizeof g_state.fp8_table);
    memcpy(fp4, g_state.fp4_table, sizeof g_state.fp4_table);
    return 0;
}

void *salt_mi355_dev_alloc(size_t nbytes) {
    void *p = nullptr;
    if (!g_state.ready || nbytes == 0) return nullptr;
    if (hip_ok(hipMalloc(&p, nbytes), "hipMalloc") != 0) return nullptr;
    return p;
}
int salt_mi355_dev_free(void *p) { return p ? hip_ok(hipFree(p), "hipFree") : 0; }
int salt_mi355_dev_upload(void *dst, const void *src, size_t nbytes) {
    return hip_ok(hipMemcpy(dst, src, nbytes, hipMemcpyHostToDevice), "hipMemcpy H2D");
}
int salt_mi355_dev_download(void *dst, const void *src, size_t nbytes) {
    return hip_ok(hipMemcpy(dst, src, nbytes, hipMemcpyDeviceToHost), "hipMemcpy D2H");
}
int salt_mi355_dev_fill(void *dst, int value, size_t nbytes) {
    return hip_ok(hipMemset(dst, value, nbytes), "hipMemset");
}
void *salt_mi355_stream(void) { return g_state.stream; }
int salt_mi355_stream_sync(void *stream) {
    return hip_ok(hipStreamSynchronize((hipStream_t)stream), "hipStreamSynchronize");
}
void *salt_mi355_event_create(void) {
    hipEvent_t e = nullptr;
    return hip_ok(hipEventCreate(&e), "hipEventCreate") == 0 ? (void *)e : nullptr;
}
int salt_mi355_event_destroy(void *e) { return hip_ok(hipEventDestroy((hipEvent_t)e), "hipEventDestroy"); }
int salt_mi355_event_record(void *e, void *stream) {
    return hip_ok(hipEventRecord((hipEvent_t)e, (hipStream_t)stream), "hipEventRecord");
}
int salt_mi355_event_elapsed_ms(void *start, void *stop, float *ms) {
    if (!ms || hip_ok(hipEventSynchronize((hipEvent_t)stop), "hipEventSynchronize") != 0) return -1;
    return hip_ok(hipEventElapsedTime(ms, (hipEvent_t)start, (hipEvent_t)stop), "hipEventElapsedTime");
}

int salt_mi355_graph_begin(void *stream) {
    return hip_ok(hipStreamBeginCapture((hipStream_t)stream, hipStreamCaptureModeThreadLocal), "hipStreamBeginCapture");
}
void *salt_mi355_graph_end(void *stream) {
    hipGraph_t graph = nullptr;
    if (hip_ok(hipStreamEndCapture((hipStream_t)stream, &graph), "hipStreamEndCapture") != 0 || !graph) return nullptr;
    hipGraphExec_t exec = nullptr;
    const int rc = hip_ok(hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0), "hipGraphInstantiate");
    (void)hipGraphDestroy(graph);
    return rc == 0 ? (void *)exec : nullptr;
}
int salt_mi355_graph_launch(void *graph_exec, void *stream) {
    return hip_ok(hipGraphLaunch((hipGraphExec_t)graph_exec, (hipStream_t)stream), "hipGraphLaunch");
}
int salt_mi355_graph_destroy(void *graph_exec) {
    return hip_ok(hipGraphExecDestroy((hipGraphExec_t)graph_exec), "hipGraphExecDestroy");
}

// ---------------------------------------------------------------- Q4, device-resident

}  // extern "C"

// Shared by the plain and the activated multi-job entry points.  activated: one token per job, whose activation row
// is gelu_tanh(xs[i]) * xs[i + act_delta].
static int q4_jobs_common(const SaltMi355Q4Job *jobs, int njobs, int C, int tokens, int chains, bool activated,
                          long long act_delta, hipStream_t stream) {
    State &s = g_state;
    if (!s.ready) { set_error("q4: library not initialised"); return -1; }
    if (!jobs || njobs < 1 || C < 1 || tokens < 1) { set_error("q4: bad arguments"); return -1; }
    if (chains != 0 && chains != 8 && chains != 4 && chains != 2) { set_error("q4: chains_per_lane %d", chains); return -1; }
    for (int j = 0; j < njobs; ++j)
        if (!jobs[j].vals || !jobs[j].scales || !jobs[j].xs || !jobs[j].ys || jobs[j].rows < 1 ||
            (size_t)jobs[j].rows > SIZE_MAX / (size_t)C) {
            set_error("q4: job %d is malformed", j);
            return -1;
        }
    std::vector<Q4Job> table((size_t)njobs);
    for (int first = 0; first < tokens; first += 4) {
        const int group = tokens - first < 4 ? tokens - first : 4;
        bool tileable = true;
        for (int j = 0; j < njobs; ++j) {
            Q4Job &q = table[(size_t)j];
            q.vals = (const uint8_t *)jobs[j].vals;
            q.scales = (const uint8_t *)jobs[j].scales;
            q.biases = (const uint8_t *)jobs[j].biases;
            q.x = jobs[j].xs + (size_t)first * (size_t)C;
            q.y = jobs[j].ys + (size_t)first * (size_t)jobs[j].rows;
            q.rows = jobs[j].rows;
            q.x_stride = C;
            q.y_stride = jobs[j].rows;
            tileable = tileable && q4_job_is_tileable(q, C);
        }
        Q4Launch launch;
        memset(&launch, 0, sizeof launch);
        launch.total_tiles = q4_assign_tiles(table.data(), njobs);
        launch.tiles_per_job = q4_uniform_tiles(table.data(), njobs);
        launch.njobs = njobs;
        launch.cols = C;
        launch.tokens = group;
        launch.code_scale = s.code_scale;
        State::TableSlot *slot = nullptr;
        if (njobs == 1) {
            launch.one = table[0];
        } else if (njobs <= Q4_INLINE_JOBS) {
            memcpy(launch.inline_jobs, table.data(), (size_t)njobs * sizeof(Q4Job));
        } else {
            slot = table_acquire(table.data(), table.size() * sizeof(Q4Job), stream);
            if (!slot) return -1;
            launch.table = (const Q4Job *)slot->device;
        }
        launch.act_delta = act_delta;
        if (activated && !tileable) { table_release(slot, stream); set_error("q4 activated: the jobs do not meet the tiled kernel's needs"); return -1; }
        const int rc = activated ? q4_activated_launch(launch, stream)
                                 : (tileable ? q4_launch(launch, chains, stream) : q4_launch_generic(launch, stream));
        table_release(slot, stream);
        if (rc != 0) { set_error("q4: kernel launch failed: %s", hipGetErrorString(hipGetLastError())); return -1; }
    }
    return 0;
}

extern "C" {

int salt_mi355_q4_jobs_dev(const SaltMi355Q4Job *jobs, int njobs, int C, int tokens, int chains, void *stream) {
    return q4_jobs_common(jobs, njobs, C, tokens, chains, false, 0, (hipStream_t)stream);
}

int salt_mi355_q4_jobs_activated_dev(const SaltMi355Q4Job *jobs, int njobs, int C, long long up_offset_floats,
                                     void *stream) {
    if (C < 64 || (C & 63) || C > MOE_FUSE_MAX_ROUTED) {
        set_error("q4 activated: C must be a multiple of 64 up to %d", MOE_FUSE_MAX_ROUTED);
        return -1;
    }
    return q4_jobs_common(jobs, njobs, C, 1, 0, true, up_offset_floats, (hipStream_t)stream);
}

// Tolerance-class decode matvec: jobs the streaming kernel cannot take (short or ragged rows, misaligned tensors)
// run on the bit-exact kernels, whose result is inside any tolerance.
int salt_mi355_q4_jobs_t_dev(const SaltMi355Q4Job *jobs, int njobs, int C, int tokens, void *stream_) {
    State &s = g_state;
    hipStream_t stream = (hipStream_t)stream_;
    if (!s.ready) { set_error("q4 t: library not initialised"); return -1; }
    if (!jobs || njobs < 1 || C < 1 || tokens < 1) { set_error("q4 t: bad arguments"); return -1; }
    bool streamable = q4_dot_takes(C) && q4_dot_tokens_per_pass(C) > 0;
    for (int j = 0; j < njobs && streamable; ++j) {
        const SaltMi355Q4Job &q = jobs[j];
        if (!q.vals || !q.scales || !q.xs || !q.ys || q.rows < 1 || (size_t)q.rows > SIZE_MAX / (size_t)C) {
            set_error("q4 t: job %d is malformed", j);
            return -1;
        }
        streamable = ((uintptr_t)q.vals & 3) == 0 && ((uintptr_t)q.scales & 1) == 0 && ((uintptr_t)q.biases & 1) == 0 &&
                     ((uintptr_t)q.xs & 3) == 0 && ((uintptr_t)q.ys & 3) == 0 &&
                     (uint64_t)DOT_BLOCK_ROWS * (uint64_t)C / 2u < (1ull << 31);
    }
    if (!streamable) return q4_jobs_common(jobs, njobs, C, tokens, 0, false, 0, stream);
    int per_pass = q4_dot_tokens_per_pass(C);
    std::vector<Q4Job> table((size_t)njobs);
    long long blocks = 0;
    for (int j = 0; j < njobs; ++j) blocks += (jobs[j].rows + DOT_BLOCK_ROWS - 1) / DOT_BLOCK_ROWS;
    // Rows too wide for the digit planes of three or four tokens at once: two column windows per block of rows keep
    // it at one read of the weights per four tokens.
    int window_waves = 0;
    if (tokens > per_pass) {
        const int want = tokens < 4 ? tokens : 4;
        window_waves = q4_dot16_window_waves(C, want, blocks);
        if (window_waves) per_pass = want;
    }
    // More tokens than one pass holds: one launch of several passes where the sixteen-row kernel serves it (the
    // passes share the weights through the cache), else a launch per pass.
    const int passes_wanted = (tokens + per_pass - 1) / per_pass;
    const int waves_passes = passes_wanted > 1 && !window_waves ? q4_dot16_waves(C, per_pass, blocks) : 0;
    const bool one_launch = waves_passes != 0 && q4_dot16_takes_passes(per_pass, waves_passes);
    for (int first = 0; first < tokens; first += one_launch ? tokens : per_pass) {
        const int group = one_launch ? per_pass : (tokens - first < per_pass ? tokens - first : per_pass);
        Q4DotLaunch launch;
        memset(&launch, 0, sizeof launch);
        const DotShape shape = q4_dot_shape(C, group, blocks);
        // the last launch of a windowed job may hold one or two tokens: those fit in one window
        const bool windowed = window_waves && group >= 3;
        const int waves16 = one_launch ? waves_passes : windowed ? q4_dot16_window_waves(C, group, blocks) : q4_dot16_waves(C, group, blocks);
        if (one_launch) { launch.passes = passes_wanted; launch.tokens_total = tokens; }
        if (windowed) launch.windows = 2;
        const int rows_per_wg = waves16 ? waves16 * 16 : shape.waves / shape.ksplit * shape.blocks_per_wave * DOT_BLOCK_ROWS;
        int wgs = 0;
        bool uniform = true;
        for (int j = 0; j < njobs; ++j) {
            Q4Job &q = table[(size_t)j];
            q.vals = (const uint8_t *)jobs[j].vals;
            q.scales = (const uint8_t *)jobs[j].scales;
            q.biases = (const uint8_t *)jobs[j].biases;
            q.x = jobs[j].xs + (size_t)first * (size_t)C;
            q.y = jobs[j].ys + (size_t)first * (size_t)jobs[j].rows;
            q.rows = jobs[j].rows;
            q.x_stride = C;
            q.y_stride = jobs[j].rows;
            q.tile0 = wgs;
            wgs += (jobs[j].rows + rows_per_wg - 1) / rows_per_wg;
            uniform = uniform && jobs[j].rows == jobs[0].rows;
        }
        launch.wgs_per_job = uniform ? wgs / njobs : 0;
        launch.njobs = njobs;
        launch.cols = C;
        launch.tokens = group;
        launch.total_wgs = wgs;
        State::TableSlot *slot = nullptr;
        if (njobs == 1) {
            launch.one = table[0];
        } else if (njobs <= Q4_INLINE_JOBS) {
            memcpy(launch.inline_jobs, table.data(), (size_t)njobs * sizeof(Q4Job));
        } else {
            slot = table_acquire(table.data(), table.size() * sizeof(Q4Job), stream);
            if (!slot) return -1;
            launch.table = (const Q4Job *)slot->device;
        }
        const int rc = waves16 ? q4_dot16_launch(launch, waves16, stream) : q4_dot_launch(launch, shape, stream);
        table_release(slot, stream);
        if (rc != 0) { set_error("q4 t: kernel launch failed: %s", hipGetErrorString(hipGetLastError())); return -1; }
    }
    return 0;
}

int salt_mi355_q4_matvec_t_dev(const void *vals, const void *scales, const void *biases, int R, int C, int B,
                               const float *xs, float *ys, void *stream) {
    SaltMi355Q4Job job;
    job.vals = vals; job.scales = scales; job.biases = biases; job.xs = xs; job.ys = ys; job.rows = R;
    return salt_mi355_q4_jobs_t_dev(&job, 1, C, B, stream);
}

int salt_mi355_q4_matvec_dev(const void *vals, const void *scales, const void *biases, int R, int C, int B,
                             const float *xs, float *ys, int chains, void *stream) {
    SaltMi355Q4Job job;
    job.vals = vals; job.scales = scales; job.biases = biases; job.xs = xs; job.ys = ys; job.rows = R;
    return salt_mi355_q4_jobs_dev(&job, 1, C, B, chains, stream);
}

}  // extern "C"
