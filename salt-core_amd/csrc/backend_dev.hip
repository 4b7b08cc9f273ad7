// Device-resident NVFP4, router and MoE entry points of libsalt_gpu_mi355.so.
#include "backend_state.h"

#include <math.h>
#include <string.h>

#include <vector>

using namespace mi355;

extern "C" {

size_t salt_mi355_q4_matmul_workspace_bytes(int C, int B) {
    if (C < 64 || (C & 63) || B < 1) return 0;
    return 3 * (size_t)B * C * 2 + (((size_t)B * (C / 64) * 4 + 255) & ~(size_t)255) + 256;
}

int salt_mi355_q4_matmul_dev(const void *vals, const void *scales, const void *biases, int R, int C, int B,
                             const float *xs, float *ys, void *workspace, void *stream) {
    if (!g_state.ready) { set_error("q4 matmul: library not initialised"); return -1; }
    if (!vals || !scales || !xs || !ys || !workspace || R < 1 || C < 64 || (C & 63) || B < 1 || B > 65535 ||
        ((uintptr_t)vals & 15) || ((uintptr_t)scales & 1) || ((uintptr_t)biases & 1) || ((uintptr_t)xs & 15) ||
        ((uintptr_t)workspace & 255)) {
        set_error("q4 matmul: bad arguments (C multiple of 64, vals / xs 16-byte and workspace 256-byte aligned)");
        return -1;
    }
    uint16_t *planes = (uint16_t *)workspace;
    const size_t plane_stride = (size_t)B * C;
    float *xsum = (float *)((uint8_t *)workspace + ((3 * plane_stride * 2 + 255) & ~(size_t)255));
    if (x_split_launch(xs, nullptr, nullptr, 1, C, B, C, planes, plane_stride, xsum, (hipStream_t)stream) != 0) {
        set_error("q4 matmul: activation split launch failed");
        return -1;
    }
    MfmaLaunch launch;
    memset(&launch, 0, sizeof launch);
    launch.one.vals = (const uint8_t *)vals; launch.one.scales = (const uint8_t *)scales;
    launch.one.biases = (const uint8_t *)biases;
    launch.one.planes = planes; launch.one.xsum = xsum; launch.one.y = ys;
    launch.one.tokens = B; launch.one.rows = R;
    launch.njobs = 1; launch.cols = C; launch.plane_stride = plane_stride;
    launch.blocks_per_wave = 0;                  // the launcher picks the tile width and counts the tiles
    if (q4_mfma_launch(launch, (hipStream_t)stream) != 0) { set_error("q4 matmul: launch failed"); return -1; }
    return 0;
}

int salt_mi355_nvfp4_qdq_dev(const float *input, int C, int B, float input_global_scale, uint8_t *packed,
                             uint8_t *scales, float *dequant, int *status_dev, void *stream) {
    if (!g_state.ready) { set_error("nvfp4 qdq: library not initialised"); return -1; }
    if (!g_state.fp8_is_ocp) { set_error("nvfp4: this device's fp8 converter is not OCP E4M3FN"); return -1; }
    if (!input || !dequant || !status_dev || C < 16 || (C & 15) || B < 1 || !isfinite(input_global_scale) ||
        input_global_scale <= 0.0f || ((uintptr_t)input & 15) || ((uintptr_t)dequant & 15) ||
        ((uintptr_t)packed & 7)) {
        set_error("nvfp4 qdq: bad arguments");
        return -1;
    }
    if (fp4_qdq_launch(input, C, B, input_global_scale, packed, scales, dequant, nullptr, status_dev,
                       (hipStream_t)stream) != 0) {
        set_error("nvfp4 qdq: launch failed");
        return -1;
    }
    return 0;
}

int salt_mi355_nvfp4_matvec_dev(const void *packed, const void *scales, float stored_divisor, int R, int C, int B,
                                const float *xs, float *ys, int chains, void *stream) {
    if (!g_state.ready) { set_error("nvfp4 matvec: library not initialised"); return -1; }
    if (!g_state.fp8_is_ocp) { set_error("nvfp4: this device's fp8 converter is not OCP E4M3FN"); return -1; }
    if (!packed || !scales || !xs || !ys || R < 1 || C < 32 || (C & 31) || B < 1 || !isfinite(stored_divisor) ||
        stored_divisor == 0.0f || ((uintptr_t)packed & 3) || ((uintptr_t)scales & 1) || ((uintptr_t)xs & 3) ||
        ((uintptr_t)ys & 3) || (chains != 0 && chains != 8 && chains != 4 && chains != 2)) {
        set_error("nvfp4 matvec: bad arguments (C must be a multiple of 32, packed 4-byte aligned)");
        return -1;
    }
    for (int first = 0; first < B; first += 4) {
        Fp4Launch launch;
        memset(&launch, 0, sizeof launch);
        launch.one.packed = (const uint8_t *)packed;
        launch.one.scales = (const uint8_t *)scales;
        launch.one.x = xs + (size_t)first * C;
        launch.one.y = ys + (size_t)first * R;
        launch.one.weight_global_scale = 1.0f / stored_divisor;
        launch.one.rows = R;
        launch.one.tile0 = 0;
        launch.one.x_stride = C;
        launch.njobs = 1;
        launch.cols = C;
        launch.tokens = B - first < 4 ? B - first : 4;
        launch.total_tiles = (R + 63) / 64;
        if (fp4_launch(launch, chains, (hipStream_t)stream) != 0) { set_error("nvfp4 matvec: launch failed"); return -1; }
    }
    return 0;
}

namespace {
// The activation pass reports per workgroup (flags) while the call is small enough for every consumer workgroup to
// read all of them; beyond that through the status word, cleared by a launch of its own.
constexpr int FP4_MATMUL_MAX_FLAGS = 4096;
struct Fp4MatmulWorkspace { int *status; int *flags; int nflags; uint16_t *plane; float *partials; size_t bytes; };
Fp4MatmulWorkspace fp4_matmul_carve(void *base, int R, int C, int B) {
    Fp4MatmulWorkspace w;
    uint8_t *p = (uint8_t *)base;
    auto take = [&](size_t n) { uint8_t *q = p; p += (n + 255) & ~(size_t)255; return q; };
    w.status = (int *)take(4);
    w.nflags = fp4_qdq_flag_count(C, B);
    if (w.nflags > FP4_MATMUL_MAX_FLAGS) w.nflags = 0;
    w.flags = w.nflags ? (int *)take((size_t)w.nflags * 4) : nullptr;
    w.plane = (uint16_t *)take((size_t)B * C * 2);
    const int splits = fp4_mfma_splits(R, C, B);
    w.partials = splits > 1 ? (float *)take((size_t)splits * B * R * 4) : nullptr;
    w.bytes = (size_t)(p - (uint8_t *)base);
    return w;
}
}  // namespace

size_t salt_mi355_nvfp4_matmul_workspace_bytes(int R, int C, int B) {
    if (R < 1 || C < 64 || (C & 63) || B < 1) return 0;
    return fp4_matmul_carve(nullptr, R, C, B).bytes;
}

int salt_mi355_nvfp4_matmul_dev(const void *packed, const void *scales, float stored_divisor, float input_global_scale,
                                int R, int C, int B, const float *xs, float *ys, int *status_dev, void *workspace,
                                void *stream) {
    if (!g_state.ready) { set_error("nvfp4 matmul: library not initialised"); return -1; }
    if (!g_state.fp8_is_ocp) { set_error("nvfp4: this device's fp8 converter is not OCP E4M3FN"); return -1; }
    if (!packed || !scales || !xs || !ys || !workspace || R < 1 || C < 64 || (C & 63) || B < 1 ||
        !isfinite(stored_divisor) || stored_divisor == 0.0f || !isfinite(input_global_scale) ||
        input_global_scale <= 0.0f || ((uintptr_t)packed & 15) || ((uintptr_t)scales & 1) || ((uintptr_t)xs & 15) ||
        ((uintptr_t)ys & 15) || ((uintptr_t)workspace & 255)) {
        set_error("nvfp4 matmul: bad arguments (C a multiple of 64; packed, xs, ys 16-byte and workspace 256-byte aligned)");
        return -1;
    }
    const Fp4MatmulWorkspace w = fp4_matmul_carve(workspace, R, C, B);
    hipStream_t s = (hipStream_t)stream;
    if (w.flags) {
        if (fp4_qdq_flags_launch(xs, C, B, input_global_scale, w.plane, w.flags, s) != 0) {
            set_error("nvfp4 matmul: activation pass failed to launch");
            return -1;
        }
    } else {
        if (clear_words_launch(w.status, 1, s) != 0) { set_error("nvfp4 matmul: status clear failed to launch"); return -1; }
        if (fp4_qdq_launch(xs, C, B, input_global_scale, nullptr, nullptr, nullptr, w.plane, w.status, s) != 0) {
            set_error("nvfp4 matmul: activation pass failed to launch");
            return -1;
        }
    }
    Fp4MfmaLaunch launch;
    memset(&launch, 0, sizeof launch);
    launch.packed = (const uint8_t *)packed; launch.scales = (const uint8_t *)scales;
    launch.plane = w.plane; launch.ys = ys; launch.partials = w.partials; launch.status = w.status;
    launch.flags = w.flags; launch.nflags = w.nflags; launch.outcome = w.status; launch.outcome_copy = status_dev;
    launch.rows = R; launch.cols = C; launch.tokens = B; launch.ksplit = fp4_mfma_splits(R, C, B);
    launch.out_scale = (1.0f / stored_divisor) / input_global_scale;
    if (fp4_mfma_launch(launch, s) != 0) { set_error("nvfp4 matmul: launch failed"); return -1; }
    if (status_dev) {
        if (w.flags) return 0;                      // the last launch has written it
        if (hip_ok(hipMemcpyAsync(status_dev, w.status, 4, hipMemcpyDeviceToDevice, s), "nvfp4 matmul status copy") != 0)
            return -1;
        return 0;
    }
    int status = -1;
    if (hip_ok(hipMemcpyAsync(&status, w.status, 4, hipMemcpyDeviceToHost, s), "nvfp4 matmul status") != 0 ||
        hip_ok(hipStreamSynchronize(s), "nvfp4 matmul sync") != 0)
        return -1;
    if (status != 0) { set_error("nvfp4 matmul: non-finite activation"); return -1; }
    return 0;
}

int salt_mi355_nvfp4_jobs_dev(const SaltMi355Fp4Job *jobs, int njobs, int C, int tokens, int chains, void *stream_handle) {
    hipStream_t stream = (hipStream_t)stream_handle;
    if (!g_state.ready) { set_error("nvfp4 jobs: library not initialised"); return -1; }
    if (!g_state.fp8_is_ocp) { set_error("nvfp4: this device's fp8 converter is not OCP E4M3FN"); return -1; }
    if (!jobs || njobs < 1 || C < 32 || (C & 31) || tokens < 1 ||
        (chains != 0 && chains != 8 && chains != 4 && chains != 2)) {
        set_error("nvfp4 jobs: bad arguments (C must be a multiple of 32)");
        return -1;
    }
    for (int j = 0; j < njobs; ++j)
        if (!jobs[j].packed || !jobs[j].scales || !jobs[j].xs || !jobs[j].ys || jobs[j].rows < 1 ||
            !isfinite(jobs[j].stored_divisor) || jobs[j].stored_divisor == 0.0f || ((uintptr_t)jobs[j].packed & 3) ||
            ((uintptr_t)jobs[j].scales & 1) || ((uintptr_t)jobs[j].xs & 3) || ((uintptr_t)jobs[j].ys & 3)) {
            set_error("nvfp4 jobs: job %d is malformed (packed 4-byte aligned, non-zero finite divisor)", j);
            return -1;
        }
    std::vector<Fp4Job> table((size_t)njobs);
    for (int first = 0; first < tokens; first += 4) {
        int tiles = 0;
        for (int j = 0; j < njobs; ++j) {
            Fp4Job &f = table[(size_t)j];
            f.packed = (const uint8_t *)jobs[j].packed;
            f.scales = (const uint8_t *)jobs[j].scales;
            f.x = jobs[j].xs + (size_t)first * C;
            f.y = jobs[j].ys + (size_t)first * jobs[j].rows;
            f.weight_global_scale = 1.0f / jobs[j].stored_divisor;
            f.rows = jobs[j].rows;
            f.tile0 = tiles;
            f.x_stride = C;
            tiles += (jobs[j].rows + 63) / 64;
        }
        Fp4Launch launch;
        memset(&launch, 0, sizeof launch);
        launch.njobs = njobs; launch.cols = C; launch.total_tiles = tiles;
        launch.tokens = tokens - first < 4 ? tokens - first : 4;
        State::TableSlot *slot = nullptr;
        if (njobs == 1) {
            launch.one = table[0];
        } else {
            slot = table_acquire(table.data(), table.size() * sizeof(Fp4Job), stream);
            if (!slot) return -1;
            launch.table = (const Fp4Job *)slot->device;
        }
        const int rc = fp4_launch(launch, chains, stream);
        table_release(slot, stream);
        if (rc != 0) { set_error("nvfp4 jobs: kernel launch failed"); return -1; }
    }
    return 0;
}

int salt_mi355_nvfp4_matvec_qdq_dev(const void *packed, const void *scales, float stored_divisor,
                                    float input_global_scale, int R, int C, const float *x, float *y, int *status_dev,
                                    int chains, void *stream) {
    if (!g_state.ready) { set_error("nvfp4 matvec: library not initialised"); return -1; }
    if (!g_state.fp8_is_ocp) { set_error("nvfp4: this device's fp8 converter is not OCP E4M3FN"); return -1; }
    if (!packed || !scales || !x || !y || !status_dev || R < 1 || C < 32 || (C & 31) || C > FP4_FUSED_MAX_COLS ||
        !isfinite(stored_divisor) || stored_divisor == 0.0f || !isfinite(input_global_scale) ||
        input_global_scale <= 0.0f || ((uintptr_t)packed & 3) || ((uintptr_t)scales & 1) || ((uintptr_t)x & 15) ||
        ((uintptr_t)y & 3) || (chains != 0 && chains != 8 && chains != 4 && chains != 2)) {
        set_error("nvfp4 matvec: bad arguments (C a multiple of 32 up to %d, packed 4-byte and x 16-byte aligned)",
                  FP4_FUSED_MAX_COLS);
        return -1;
    }
    Fp4Launch launch;
    memset(&launch, 0, sizeof launch);
    launch.one.packed = (const uint8_t *)packed;
    launch.one.scales = (const uint8_t *)scales;
    launch.one.x = x;
    launch.one.y = y;
    launch.one.weight_global_scale = 1.0f / stored_divisor;
    launch.one.rows = R;
    launch.one.x_stride = C;
    launch.njobs = 1; launch.cols = C; launch.tokens = 1;
    launch.total_tiles = (R + 63) / 64;
    launch.qdq = 1; launch.input_global_scale = input_global_scale; launch.status = status_dev;
    if (fp4_launch(launch, chains, (hipStream_t)stream) != 0) { set_error("nvfp4 matvec: launch failed"); return -1; }
    return 0;
}

// Tolerance-class reference matvec: jobs of `tokens` raw activation rows each, quantised inside the launch.
int salt_mi355_nvfp4_jobs_t_dev(const SaltMi355Fp4Job *jobs, int njobs, int C, int tokens, float input_global_scale,
                                int *status_dev, void *stream_handle) {
    hipStream_t stream = (hipStream_t)stream_handle;
    if (!g_state.ready) { set_error("nvfp4 t: library not initialised"); return -1; }
    if (!g_state.fp8_is_ocp) { set_error("nvfp4: this device's fp8 converter is not OCP E4M3FN"); return -1; }
    if (!jobs || njobs < 1 || tokens < 1 || !status_dev || !isfinite(input_global_scale) || input_global_scale <= 0.0f ||
        C < 32 || (C & 31) || C > FP4_FUSED_MAX_COLS) {
        set_error("nvfp4 t: bad arguments (C a multiple of 32 up to %d, a status word)", FP4_FUSED_MAX_COLS);
        return -1;
    }
    bool streamable = fp4_dot_takes(C);
    for (int j = 0; j < njobs; ++j) {
        const SaltMi355Fp4Job &f = jobs[j];
        if (!f.packed || !f.scales || !f.xs || !f.ys || f.rows < 1 || !isfinite(f.stored_divisor) ||
            f.stored_divisor == 0.0f || ((uintptr_t)f.packed & 3) || ((uintptr_t)f.scales & 1) || ((uintptr_t)f.xs & 15) ||
            ((uintptr_t)f.ys & 3)) {
            set_error("nvfp4 t: job %d is malformed (packed 4-byte, activations 16-byte aligned, non-zero finite divisor)", j);
            return -1;
        }
    }
    if (!streamable) {
        // column counts the streaming kernel does not take run on the bit-exact one-launch kernel, token by token
        for (int j = 0; j < njobs; ++j)
            for (int t = 0; t < tokens; ++t)
                if (salt_mi355_nvfp4_matvec_qdq_dev(jobs[j].packed, jobs[j].scales, jobs[j].stored_divisor, input_global_scale,
                                                    jobs[j].rows, C, jobs[j].xs + (size_t)t * C,
                                                    jobs[j].ys + (size_t)t * jobs[j].rows, status_dev, 0, stream_handle) != 0)
                    return -1;
        return 0;
    }
    std::vector<Fp4Job> table((size_t)njobs);
    for (int first = 0; first < tokens; first += 4) {
        const int group = tokens - first < 4 ? tokens - first : 4;
        long long blocks = 0;
        for (int j = 0; j < njobs; ++j) blocks += (jobs[j].rows + DOT_BLOCK_ROWS - 1) / DOT_BLOCK_ROWS;
        const DotShape shape = fp4_dot_shape(C, group, blocks);
        const int rows_per_wg = shape.waves / shape.ksplit * DOT_BLOCK_ROWS;
        Fp4DotLaunch launch;
        memset(&launch, 0, sizeof launch);
        int wgs = 0;
        bool uniform = true;
        for (int j = 0; j < njobs; ++j) {
            Fp4Job &f = table[(size_t)j];
            f.packed = (const uint8_t *)jobs[j].packed;
            f.scales = (const uint8_t *)jobs[j].scales;
            f.x = jobs[j].xs + (size_t)first * C;
            f.y = jobs[j].ys + (size_t)first * jobs[j].rows;
            f.weight_global_scale = 1.0f / jobs[j].stored_divisor;
            f.rows = jobs[j].rows;
            f.tile0 = wgs;
            f.x_stride = C;
            wgs += (jobs[j].rows + rows_per_wg - 1) / rows_per_wg;
            uniform = uniform && jobs[j].rows == jobs[0].rows;
        }
        launch.njobs = njobs; launch.cols = C; launch.tokens = group; launch.total_wgs = wgs;
        launch.wgs_per_job = uniform ? wgs / njobs : 0;
        launch.input_global_scale = input_global_scale;
        launch.status = status_dev;
        State::TableSlot *slot = nullptr;
        if (njobs == 1) {
            launch.one = table[0];
        } else {
            slot = table_acquire(table.data(), table.size() * sizeof(Fp4Job), stream);
            if (!slot) return -1;
            launch.table = (const Fp4Job *)slot->device;
        }
        const int rc = fp4_dot_launch(launch, shape, stream);
        table_release(slot, stream);
        if (rc != 0) { set_error("nvfp4 t: kernel launch failed: %s", hipGetErrorString(hipGetLastError())); return -1; }
    }
    return 0;
}

int salt_mi355_nvfp4_matvec_t_dev(const void *packed, const void *scales, float stored_divisor, float input_global_scale,
                                  int R, int C, int B, const float *xs, float *ys, int *status_dev, void *stream) {
    SaltMi355Fp4Job job;
    job.packed = packed; job.scales = scales; job.stored_divisor = stored_divisor; job.xs = xs; job.ys = ys; job.rows = R;
    return salt_mi355_nvfp4_jobs_t_dev(&job, 1, C, B, input_global_scale, status_dev, stream);
}

int salt_mi355_bf16_matvec_dev(const void *weights, int R, int C, int B, const float *xs, const float *bias, float *ys,
                                void *stream) {
    if (!g_state.ready) { set_error("bf16 matvec: library not initialised"); return -1; }
    if (!weights || !xs || !ys || R < 1 || C < 1 || B < 1 || ((uintptr_t)xs & 3) || ((uintptr_t)ys & 3) ||
        ((uintptr_t)bias & 3)) {
        set_error("bf16 matvec: bad arguments");
        return -1;
    }
    Bf16Launch launch;
    launch.weights = (const uint16_t *)weights;
    launch.x = xs; launch.bias = bias; launch.y = ys;
    launch.rows = R; launch.cols = C; launch.tokens = B;
    launch.x_stride = C; launch.y_stride = R;
    if (bf16_launch(launch, (hipStream_t)stream) != 0) { set_error("bf16 matvec: launch failed"); return -1; }
    return 0;
}

int salt_mi355_q8_matvec_dev(const void *vals, const void *scales, const void *biases, int R, int C, int B,
                              const float *xs, float *ys, void *stream) {
    if (!g_state.ready) { set_error("q8 matvec: library not initialised"); return -1; }
    if (!vals || !scales || !xs || !ys || R < 1 || C < 1 || B < 1 || B > 65535 || ((uintptr_t)xs & 3) ||
        ((uintptr_t)ys & 3)) {
        set_error("q8 matvec: bad arguments");
        return -1;
    }
    Q8Launch launch;
    launch.vals = (const uint8_t *)vals; launch.scales = (const uint8_t *)scales; launch.biases = (const uint8_t *)biases;
    launch.x = xs; launch.y = ys;
    launch.rows = R; launch.cols = C; launch.tokens = B;
    launch.x_stride = C; launch.y_stride = R;
    if (q8_launch(launch, (hipStream_t)stream) != 0) { set_error("q8 matvec: launch failed"); return -1; }
    return 0;
}

int salt_mi355_cells_dev(const SaltMi355Cell *cells, int count, int *status_dev, void *stream_handle) {
    hipStream_t stream = (hipStream_t)stream_handle;
    if (!g_state.ready) { set_error("cells: library not initialised"); return -1; }
    if (!cells || count < 1 || !status_dev) { set_error("cells: bad arguments"); return -1; }
    for (int c = 0; c < count; ++c) {
        const SaltMi355Cell &cell = cells[c];
        const void *const *v = cell.views;
        const int n = (int)cell.n;
        int need = 0, rc = -1;
        switch (cell.kind) {
        case 1: need = 3; break;
        case 2: need = 4; break;
        case 3: need = 4; break;
        case 4: need = 8; break;
        case 5: need = 1; break;
        case 6: need = 3; break;
        default: set_error("cells: cell %d has unknown kind %d", c, cell.kind); return -1;
        }
        bool ok = cell.n >= 1 && (cell.kind == 5 || cell.n <= 0x7fffffffu);
        for (int k = 0; k < need; ++k)
            ok = ok && (v[k] || (cell.kind == 1 && k == 1 && cell.aux == 0)) && ((uintptr_t)v[k] & 3) == 0;
        if (!ok) { set_error("cells: cell %d has a null or misaligned view, or n = 0", c); return -1; }
        switch (cell.kind) {
        case 1:
            if (cell.aux > 1) { set_error("cells: rmsnorm aux must be 0 or 1"); return -1; }
            rc = norm_cell_launch(0, (const float *)v[0], cell.aux ? (const float *)v[1] : nullptr, nullptr, (float *)v[2], n,
                                  cell.eps, 0.0f, status_dev, stream);
            break;
        case 2:
            if (cell.aux < 1 || cell.aux > cell.n) { set_error("cells: topk aux must be in [1, n]"); return -1; }
            rc = router_topk_launch((const float *)v[0], (const float *)v[1], n, (int)cell.aux, 1, (int *)v[2], (float *)v[3],
                                    status_dev + 1, stream);
            if (rc == 0) rc = merge_status_launch(status_dev, status_dev + 1, stream);
            break;
        case 3:
            rc = norm_cell_launch(2, (const float *)v[1], (const float *)v[2], (const float *)v[0], (float *)v[3], n, cell.eps,
                                  0.0f, status_dev, stream);
            break;
        case 4:
            rc = combine_cell_launch((const float *)v[0], (const float *)v[1], (const float *)v[2], (const float *)v[3],
                                     (const float *)v[4], (const float *)v[5], (float *)v[6], (float *)v[7], n, cell.eps,
                                     cell.scalar, status_dev, nullptr, nullptr, nullptr, 0, stream);
            break;
        case 5:
            rc = softcap_cell_launch((float *)v[0], cell.n, cell.scalar, status_dev, stream);
            break;
        case 6:
            rc = norm_cell_launch(1, (const float *)v[0], (const float *)v[1], nullptr, (float *)v[2], n, cell.eps, cell.scalar,
                                  status_dev, stream);
            break;
        }
        if (rc != 0) { set_error("cells: cell %d (kind %d) was refused or failed to launch", c, cell.kind); return -1; }
    }
    return 0;
}

namespace {

struct FfnWorkspace {
    float *norm_a, *norm_b, *router_in, *dense_out, *routed_out, *sum, *gate, *up, *act, *logits, *expert_out;
    void *moe;
};

size_t pad256(size_t n) { return (n + 255) & ~(size_t)255; }

size_t ffn_carve(const SaltMi355FfnLayer &L, void *base, FfnWorkspace *ws) {
    uint8_t *p = (uint8_t *)base;
    const size_t H = (size_t)L.hidden * 4, D = (size_t)L.dense * 4;
    auto take = [&](size_t bytes) { uint8_t *at = p; p += pad256(bytes); return at; };
    FfnWorkspace w;
    w.norm_a = (float *)take(H); w.norm_b = (float *)take(H); w.router_in = (float *)take(H);
    w.dense_out = (float *)take(H); w.routed_out = (float *)take(H); w.sum = (float *)take(2 * H);
    w.gate = (float *)take(D); w.up = (float *)take(D); w.act = (float *)take(D);
    w.logits = (float *)take((size_t)L.n_experts * 4);
    w.expert_out = (float *)take((size_t)L.topk * H);
    w.moe = take(moe_workspace_bytes(MoeGeometry{L.hidden, L.routed, L.n_experts, L.topk}));
    if (ws) *ws = w;
    return (size_t)(p - (uint8_t *)base);
}

bool ffn_layer_ok(const SaltMi355FfnLayer *L) {
    if (!L || L->hidden < 64 || (L->hidden & 63) || L->routed < 64 || (L->routed & 63) || L->dense < 64 || (L->dense & 63) ||
        L->n_experts < 1 || L->topk < 1 || L->topk > L->n_experts)
        return false;
    const void *need[] = {L->pre_norm, L->pre_norm_2, L->router_scale, L->per_expert_scale, L->post_norm_1, L->post_norm_2,
                          L->post_norm, L->dense_gate[0], L->dense_gate[1], L->dense_up[0], L->dense_up[1],
                          L->dense_down[0], L->dense_down[1], L->router[0], L->router[1], L->pool};
    for (const void *q : need)
        if (!q) return false;
    const size_t n = (size_t)L->hidden * (size_t)L->routed;
    return ((uintptr_t)L->pool & 3) == 0 && (L->expert_stride & 15) == 0 && L->expert_stride >= 3 * (n / 2 + 4 * (n / 64));
}

}  // namespace

size_t salt_mi355_ffn_block_workspace_bytes(const SaltMi355FfnLayer *layer) {
    return ffn_layer_ok(layer) ? ffn_carve(*layer, nullptr, nullptr) : 0;
}

int salt_mi355_ffn_block_dev(const SaltMi355FfnLayer *layer, const float *residual, float *out, int *selected,
                             float *weights, int *status_dev, void *workspace, void *stream_handle) {
    hipStream_t stream = (hipStream_t)stream_handle;
    if (!g_state.ready) { set_error("ffn block: library not initialised"); return -1; }
    if (!ffn_layer_ok(layer) || !residual || !out || !selected || !weights || !status_dev || !workspace ||
        ((uintptr_t)workspace & 255) || residual == out) {
        set_error("ffn block: bad arguments (hidden, dense, routed multiples of 64; workspace 256-byte aligned)");
        return -1;
    }
    const SaltMi355FfnLayer &L = *layer;
    FfnWorkspace ws;
    ffn_carve(L, workspace, &ws);
    const MoeGeometry g = {L.hidden, L.routed, L.n_experts, L.topk};
    MoeWorkspace moe;
    moe_workspace_carve(g, ws.moe, &moe);

    // dense gate and up as one two-job launch; the job records travel inside that launch's arguments
    Q4Job dense[2];
    memset(dense, 0, sizeof dense);
    for (int k = 0; k < 2; ++k) {
        const void *const *t = k == 0 ? L.dense_gate : L.dense_up;
        dense[k].vals = (const uint8_t *)t[0]; dense[k].scales = (const uint8_t *)t[1]; dense[k].biases = (const uint8_t *)t[2];
        dense[k].x = ws.norm_a; dense[k].y = k == 0 ? ws.gate : ws.up;
        dense[k].rows = L.dense; dense[k].x_stride = L.hidden; dense[k].y_stride = L.dense;
    }
    Q4Launch gate_up;
    memset(&gate_up, 0, sizeof gate_up);
    gate_up.total_tiles = q4_assign_tiles(dense, 2);
    gate_up.tiles_per_job = q4_uniform_tiles(dense, 2);
    memcpy(gate_up.inline_jobs, dense, sizeof dense);
    gate_up.table = nullptr; gate_up.njobs = 2; gate_up.cols = L.hidden; gate_up.tokens = 1;
    gate_up.code_scale = g_state.code_scale;
    const bool tileable = q4_job_is_tileable(dense[0], L.hidden) && q4_job_is_tileable(dense[1], L.hidden);

    if (ffn_pre_launch(residual, L.pre_norm, L.pre_norm_2, L.router_scale, ws.norm_a, ws.norm_b, ws.router_in, L.hidden, L.eps,
                       status_dev, stream) != 0) {
        set_error("ffn block: pre-norm launch failed");
        return -1;
    }
    // The dense branch runs beside the routed one on the library's second stream.
    hipStream_t side = g_state.side;
    if (hip_ok(hipEventRecord(g_state.fork, stream), "ffn block fork") != 0 ||
        hip_ok(hipStreamWaitEvent(side, g_state.fork, 0), "ffn block fork wait") != 0)
        return -1;
    int rc = tileable ? q4_launch(gate_up, 0, side) : q4_launch_generic(gate_up, side);
    if (rc == 0) rc = moe_activate_launch(ws.gate, ws.up, ws.act, (size_t)L.dense, side);
    if (rc == 0)
        rc = salt_mi355_q4_matvec_dev(L.dense_down[0], L.dense_down[1], L.dense_down[2], L.hidden, L.dense, 1, ws.act,
                                      ws.dense_out, 0, side);
    // the join is recorded even after a failure, so that the caller's stream never outruns the side stream
    const int recorded = hip_ok(hipEventRecord(g_state.join, side), "ffn block join");
    if (rc != 0 || recorded != 0) {
        (void)hipStreamWaitEvent(stream, g_state.join, 0);
        set_error("ffn block: dense branch failed to launch");
        return -1;
    }

    // routed branch; a rejected residual leaves its inputs unwritten: the router then works on whatever they held,
    // which it either rejects or routes harmlessly, and the combine publishes nothing in both cases
    if (salt_mi355_q8_matvec_dev(L.router[0], L.router[1], L.router[2], L.n_experts, L.hidden, 1, ws.router_in, ws.logits,
                                 stream) != 0)
        return -1;
    if (moe_decode_step_launch(g, (const uint8_t *)L.pool, L.expert_stride, ws.logits, L.per_expert_scale, ws.norm_b,
                               selected, weights, ws.expert_out, nullptr, moe, g_state.code_scale, stream) != 0) {
        set_error("ffn block: unsupported MoE geometry or launch failure");
        return -1;
    }
    if (hip_ok(hipStreamWaitEvent(stream, g_state.join, 0), "ffn block join wait") != 0) return -1;
    if (combine_cell_launch(residual, ws.dense_out, ws.routed_out, L.post_norm_1, L.post_norm_2, L.post_norm, ws.sum, out,
                            L.hidden, L.eps, L.layer_scalar, status_dev, moe.status, ws.expert_out, weights, L.topk,
                            stream) != 0) {
        set_error("ffn block: combine launch failed");
        return -1;
    }
    return 0;
}

int salt_mi355_router_topk_dev(const float *logits, const float *per_expert_scale, int n_experts, int topk,
                               int sorted_by_id, int *selected, float *weights, int *status_dev, void *stream) {
    if (!g_state.ready) { set_error("router: library not initialised"); return -1; }
    if (!logits || !per_expert_scale || !selected || !weights || !status_dev) { set_error("router: null argument"); return -1; }
    if (router_topk_launch(logits, per_expert_scale, n_experts, topk, sorted_by_id, selected, weights, status_dev,
                           (hipStream_t)stream) != 0) {
        set_error("router: unsupported geometry (experts %d, topk %d) or launch failure", n_experts, topk);
        return -1;
    }
    return 0;
}

size_t salt_mi355_moe_prefill_workspace_bytes(int hidden, int routed, int n_experts, int topk, int tokens) {
    if (hidden < 64 || routed < 64 || n_experts < 1 || topk < 1 || tokens < 1) return 0;
    const MoeGeometry g = {hidden, routed, n_experts, topk};
    return moe_prefill_workspace_bytes(g, tokens);
}

int salt_mi355_moe_prefill_dev(const void *pool, size_t expert_stride, int hidden, int routed, int n_experts, int topk,
                               int tokens, const int *selected, const float *weights, const float *inputs,
                               float *outputs, int *group_rows, int *row_pairs, int *status_dev, void *workspace,
                               void *stream) {
    if (!g_state.ready) { set_error("moe prefill: library not initialised"); return -1; }
    if (!pool || !selected || !weights || !inputs || !outputs || !workspace || ((uintptr_t)pool & 15) ||
        (expert_stride & 15) || ((uintptr_t)workspace & 255) || ((uintptr_t)inputs & 15)) {
        set_error("moe prefill: bad arguments (pool, stride and inputs 16-byte aligned, workspace 256-byte aligned)");
        return -1;
    }
    const MoeGeometry g = {hidden, routed, n_experts, topk};
    const size_t n = (size_t)hidden * (size_t)routed;
    if (hidden < 64 || (hidden & 63) || routed < 64 || (routed & 63) || expert_stride < 3 * (n / 2 + 4 * (n / 64))) {
        set_error("moe prefill: hidden and routed must be multiples of 64 and the stride must cover a slot");
        return -1;
    }
    if (moe_prefill_launch(g, (const uint8_t *)pool, expert_stride, tokens, selected, weights, inputs, outputs,
                           group_rows, row_pairs, status_dev, workspace, (hipStream_t)stream) != 0) {
        set_error("moe prefill: unsupported geometry (experts %d, topk %d, tokens %d) or launch failure", n_experts,
                  topk, tokens);
        return -1;
    }
    if (status_dev) return 0;
    // no status word from the caller: wait, and report an invalid selection as a failed call
    int status = -1;
    if (hip_ok(hipMemcpyAsync(&status, workspace, sizeof status, hipMemcpyDeviceToHost, (hipStream_t)stream),
               "moe prefill status") != 0 ||
        hip_ok(hipStreamSynchronize((hipStream_t)stream), "moe prefill sync") != 0)
        return -1;
    if (status != 0) { set_error("moe prefill: invalid selection (expert id, duplicate or weight)"); return -1; }
    return 0;
}

size_t salt_mi355_moe_workspace_bytes(int hidden, int routed, int n_experts, int topk) {
    if (hidden < 1 || routed < 1 || n_experts < 1 || topk < 1) return 0;
    const MoeGeometry g = {hidden, routed, n_experts, topk};
    return moe_workspace_bytes(g);
}

int salt_mi355_moe_decode_step_dev(const void *pool, size_t expert_stride, int hidden, int routed, int n_experts,
                                   int topk, const float *logits, const float *per_expert_scale, const float *x,
                                   int *selected, float *weights, float *expert_out, float *out, void *workspace,
                                   void *stream) {
    if (!g_state.ready) { set_error("moe step: library not initialised"); return -1; }
    if (!pool || !logits || !per_expert_scale || !x || !selected || !weights || !out || !workspace ||
        ((uintptr_t)pool & 3) || (expert_stride & 15) || ((uintptr_t)workspace & 255)) {
        set_error("moe step: bad arguments (pool 4-byte aligned, expert stride a multiple of 16, workspace 256-byte aligned)");
        return -1;
    }
    const MoeGeometry g = {hidden, routed, n_experts, topk};
    const size_t n = (size_t)hidden * (size_t)routed;
    if (hidden < 64 || (hidden & 63) || routed < 64 || (routed & 63) || expert_stride < 3 * (n / 2 + 4 * (n / 64))) {
        set_error("moe step: hidden and routed must be multiples of 64 and the stride must cover a slot");
        return -1;
    }
    MoeWorkspace ws;
    moe_workspace_carve(g, workspace, &ws);
    if (moe_decode_step_launch(g, (const uint8_t *)pool, expert_stride, logits, per_expert_scale, x, selected, weights,
                               expert_out, out, ws, g_state.code_scale, (hipStream_t)stream) != 0) {
        set_error("moe step: unsupported geometry or launch failure");
        return -1;
    }
    return 0;
}

// Tolerance-class form of the step: the projections run on the streaming kernel; geometries it does not serve take
// the bit-exact plan (whose result is inside any tolerance).
int salt_mi355_moe_decode_step_t_dev(const void *pool, size_t expert_stride, int hidden, int routed, int n_experts,
                                     int topk, const float *logits, const float *per_expert_scale, const float *x,
                                     int *selected, float *weights, float *expert_out, float *out, void *workspace,
                                     void *stream) {
    if (!g_state.ready) { set_error("moe step t: library not initialised"); return -1; }
    if (!pool || !logits || !per_expert_scale || !x || !selected || !weights || !out || !workspace ||
        ((uintptr_t)pool & 3) || (expert_stride & 15) || ((uintptr_t)workspace & 255)) {
        set_error("moe step t: bad arguments (pool 4-byte aligned, expert stride a multiple of 16, workspace 256-byte aligned)");
        return -1;
    }
    const MoeGeometry g = {hidden, routed, n_experts, topk};
    const size_t n = (size_t)hidden * (size_t)routed;
    if (hidden < 64 || (hidden & 63) || routed < 64 || (routed & 63) || n_experts < 1 || topk < 1 || topk > n_experts ||
        expert_stride < 3 * (n / 2 + 4 * (n / 64))) {
        set_error("moe step t: hidden and routed must be multiples of 64 and the stride must cover a slot");
        return -1;
    }
    MoeWorkspace ws;
    moe_workspace_carve(g, workspace, &ws);
    const int served = moe_decode_step_t_launch(g, (const uint8_t *)pool, expert_stride, logits, per_expert_scale, x,
                                                selected, weights, expert_out, out, ws, (hipStream_t)stream);
    if (served == 0) return 0;
    if (served != MOE16_NOT_SERVED) {
        set_error("moe step t: a launch failed: %s", hipGetErrorString(hipGetLastError()));
        return -1;
    }
    // a geometry the streaming kernels do not take: the bit-exact plan, whose result is inside any tolerance
    return salt_mi355_moe_decode_step_dev(pool, expert_stride, hidden, routed, n_experts, topk, logits, per_expert_scale,
                                          x, selected, weights, expert_out, out, workspace, stream);
}

// ---------------------------------------------------------------- policy

int salt_mi355_set_tolerance_class(int enabled) {
    const int before = g_state.tolerance_class;
    g_state.tolerance_class = enabled != 0;
    return before;
}

// ---------------------------------------------------------------- launch skeleton (measurement aid)

}  // extern "C"

namespace {
__global__ void skeleton_kernel(int *never) {
    if (never && threadIdx.x == 0x7fffffff) *never = 1;       // nothing
}
}  // namespace

extern "C" {

int salt_mi355_launch_skeleton_dev(int workgroups_a, int threads_a, int lds_bytes_a, int workgroups_b, int threads_b,
                                   int lds_bytes_b, void *stream) {
    if (!g_state.ready) { set_error("launch skeleton: library not initialised"); return -1; }
    const int shapes[2][3] = {{workgroups_a, threads_a, lds_bytes_a}, {workgroups_b, threads_b, lds_bytes_b}};
    static int raised = 0;
    for (const int (&shape)[3] : shapes) {
        if (shape[0] == 0) continue;
        if (shape[0] < 0 || shape[1] < 1 || shape[1] > 1024 || shape[2] < 0 || shape[2] > DOT_LDS_LIMIT) {
            set_error("launch skeleton: bad shape");
            return -1;
        }
        if (shape[2] > raised) {
            if (hip_ok(hipFuncSetAttribute((const void *)skeleton_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, shape[2]),
                       "hipFuncSetAttribute") != 0)
                return -1;
            raised = shape[2];
        }
        hipLaunchKernelGGL(skeleton_kernel, dim3(shape[0]), dim3(shape[1]), shape[2], (hipStream_t)stream, (int *)nullptr);
        if (hip_ok(hipGetLastError(), "skeleton launch") != 0) return -1;
    }
    return 0;
}

// ---------------------------------------------------------------- the same step without a workspace argument

}  // extern "C"

// The workspace of salt_mi355_moe_decode_step_static_dev: one array per device for as long as the process lives.  In
// host code this name is only a handle for hipGetSymbolAddress; the address the kernels use is looked up once per
// device and kept below.
static __device__ __align__(256) unsigned char moe_static_scratch[SALT_MI355_MOE_STATIC_SCRATCH_BYTES];
static void *moe_static_scratch_address[16];        // by device ordinal; nullptr = not looked up yet

static void *moe_static_scratch_of_current_device();

namespace mi355 {
// Called by salt_mi355_init on the device it initialises: the entry point then finds the address without a runtime
// query (one that could load the code object in the middle of a capture or a serving loop).
int moe_static_scratch_prepare() { return moe_static_scratch_of_current_device() ? 0 : -1; }
}  // namespace mi355

static void *moe_static_scratch_of_current_device() {
    int device = -1;
    if (hip_ok(hipGetDevice(&device), "hipGetDevice") != 0) return nullptr;
    if (device < 0 || device >= 16) { set_error("moe static step: device ordinal %d is out of range", device); return nullptr; }
    if (!moe_static_scratch_address[device]) {
        void *address = nullptr;
        if (hip_ok(hipGetSymbolAddress(&address, HIP_SYMBOL(moe_static_scratch)), "hipGetSymbolAddress") != 0 || !address)
            return nullptr;
        moe_static_scratch_address[device] = address;
    }
    return moe_static_scratch_address[device];
}

extern "C" {

int salt_mi355_moe_decode_step_static_dev(const void *pool, size_t expert_stride, int hidden, int routed, int n_experts,
                                          int topk, const float *logits, const float *per_expert_scale, const float *x,
                                          int *selected, float *weights, float *expert_out, float *out,
                                          int *status_dev, void *stream) {
    if (!g_state.ready) { set_error("moe static step: library not initialised"); return -1; }
    if (hidden < 1 || routed < 1 || n_experts < 1 || topk < 1) { set_error("moe static step: bad geometry"); return -1; }
    const size_t need = salt_mi355_moe_workspace_bytes(hidden, routed, n_experts, topk);
    if (need == 0 || need > (size_t)SALT_MI355_MOE_STATIC_SCRATCH_BYTES) {
        set_error("moe static step: this geometry needs %zu bytes of workspace, the static one holds %d", need,
                  SALT_MI355_MOE_STATIC_SCRATCH_BYTES);
        return -1;
    }
    void *scratch = moe_static_scratch_of_current_device();
    if (!scratch) return -1;
    if (!pool || !logits || !per_expert_scale || !x || !selected || !weights || !out || ((uintptr_t)pool & 3) ||
        (expert_stride & 15)) {
        set_error("moe static step: bad arguments (pool 4-byte aligned, expert stride a multiple of 16)");
        return -1;
    }
    const MoeGeometry g = {hidden, routed, n_experts, topk};
    const size_t n = (size_t)hidden * (size_t)routed;
    if (hidden < 64 || (hidden & 63) || routed < 64 || (routed & 63) || expert_stride < 3 * (n / 2 + 4 * (n / 64))) {
        set_error("moe static step: hidden and routed must be multiples of 64 and the stride must cover a slot");
        return -1;
    }
    MoeWorkspace ws;
    moe_workspace_carve(g, scratch, &ws);
    // Every word of the workspace that a launch reads is written earlier in the same step (the status word by the
    // router, the job tables and the intermediate vectors by their producers, the tile counters of the ordered sum by
    // the first launch): nothing has to start at zero.
    if (status_dev) ws.status = status_dev;
    if (moe_decode_step_launch(g, (const uint8_t *)pool, expert_stride, logits, per_expert_scale, x, selected, weights,
                               expert_out, out, ws, g_state.code_scale, (hipStream_t)stream) != 0) {
        set_error("moe static step: unsupported geometry or launch failure");
        return -1;
    }
    return 0;
}

int salt_mi355_q4_decode_dev(const void *vals, const void *scales, const void *biases, size_t n, float *out, void *stream) {
    if (!g_state.ready) { set_error("q4 decode: library not initialised"); return -1; }
    if (!vals || !scales || !out || ((uintptr_t)out & 3)) { set_error("q4 decode: bad arguments"); return -1; }
    if (q4_decode_launch((const uint8_t *)vals, (const uint8_t *)scales, (const uint8_t *)biases, n, out, (hipStream_t)stream) != 0) {
        set_error("q4 decode: launch failed");
        return -1;
    }
    return 0;
}

int salt_mi355_nvfp4_dequant_weights_dev(const void *packed, const void *scales, float stored_divisor, int R, int C,
                                         float *out, void *stream) {
    if (!g_state.ready) { set_error("nvfp4 dequant: library not initialised"); return -1; }
    if (!g_state.fp8_is_ocp) { set_error("nvfp4: this device's fp8 converter is not OCP E4M3FN"); return -1; }
    if (!packed || !scales || !out || R < 1 || C < 16 || (C & 15) || !isfinite(stored_divisor) || stored_divisor == 0.0f ||
        ((uintptr_t)out & 3)) {
        set_error("nvfp4 dequant: bad arguments (C a multiple of 16, non-zero finite divisor)");
        return -1;
    }
    if (nvfp4_dequant_launch((const uint8_t *)packed, (const uint8_t *)scales, 1.0f / stored_divisor, R, C, out,
                             (hipStream_t)stream) != 0) {
        set_error("nvfp4 dequant: launch failed");
        return -1;
    }
    return 0;
}

int salt_mi355_router_fixture_dev(int n_experts, int topk, uint64_t state, int layer, double locality, int *idx, float *w,
                                  void *stream) {
    if (!g_state.ready) { set_error("fixture router: library not initialised"); return -1; }
    if (!idx || !w || router_fixture_launch(n_experts, topk, state, layer, locality, idx, w, (hipStream_t)stream) != 0) {
        set_error("fixture router: bad arguments (1 <= topk <= n_experts <= 1024)");
        return -1;
    }
    return 0;
}

int salt_mi355_moe_activate_dev(const float *gate, const float *up, float *act, size_t n, void *stream) {
    if (!g_state.ready || !gate || !up || !act || n < 1) { set_error("moe activate: bad arguments"); return -1; }
    return moe_activate_launch(gate, up, act, n, (hipStream_t)stream);
}

int salt_mi355_moe_reduce_dev(const float *expert_out, const float *weights, int topk, int hidden, float *out,
                              void *stream) {
    if (!g_state.ready || !expert_out || !weights || !out || topk < 1 || hidden < 1) {
        set_error("moe reduce: bad arguments");
        return -1;
    }
    return moe_reduce_launch(expert_out, weights, topk, hidden, out, nullptr, (hipStream_t)stream);
}

}  // extern "C"
