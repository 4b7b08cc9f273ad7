// The engine-facing entry points (salt_gpu_*) of libsalt_gpu_mi355.so: host
// pointers in, host pointers out, weights addressed through described
// resources that are kept resident in HBM.  Each entry point validates, maps
// host weight pointers to their HBM copies, stages activations through pinned
// memory, runs the device-resident kernels and publishes outputs either at
// once or, in defer mode, at salt_gpu_sync().
//
// Behaviour follows the reference HIP backend where the engine depends on it
// (reference src/gpu_hip.cpp:3681-3760 init/requirements, 4176-4462 resource
// lifecycle, 4464-4575 projections, 5987-6432 MoE chain, 6434-6680 expert
// seats, 804-1025 residency operations); the implementation is this library's
// own.
#include "backend_state.h"

#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <algorithm>
#include <unordered_map>
#include <vector>

using namespace mi355;

namespace {

constexpr uint32_t KIND_MAX = 2;                 // arena, trunk, expert layer (reference gpu_resource.h:9-13)
constexpr uint32_t KIND_EXPERT_LAYER = 2;
constexpr int MAX_C = 8192;                      // capacities published like the reference (gpu_hip.cpp:21-28)
constexpr uint32_t MAX_OUTPUT_FLOATS = 4096u * 2816u;
constexpr uint32_t MAX_BATCH_JOBS = 4096;
constexpr uint32_t SHARED_SLOTS = 8;
constexpr int MAX_PROJ_BATCH = 512;

struct Resource {
    uint32_t kind = 0, id = 0;
    const uint8_t *host = nullptr;
    size_t nbytes = 0;
    uint8_t *device = nullptr;        // whole-resource HBM copy
    int active = 0;
    int policy = 0;
    uint64_t window_offset = 0;       // bounded-window policy: the one bound window
    size_t window_bytes = 0;
    uint8_t *window_device = nullptr;
    int pool = 0;                     // pool-bound: only the bytes its tensors occupy become resident
};

// One merged byte range of a pool-bound resource that registered tensors occupy
// (reference gpu_hip.cpp:3212-3340).  It is resident either inside the residency
// arena (a permanent span) or in an allocation of its own.
struct Region {
    int resource = -1;
    const uint8_t *host = nullptr;
    size_t nbytes = 0;
    uint64_t source_offset = 0;       // of `host` inside the resource
    uint64_t arena_offset = 0;        // inside the residency arena, once laid out
    size_t populated = 0;             // bytes of the span copied so far
    uint8_t *device = nullptr;        // set when the range is readable by kernels
    uint8_t *owned = nullptr;         // allocation of its own (no residency arena)
};

struct Tensor {
    int resource = -1;                // index into resources
    const uint8_t *vals = nullptr, *scales = nullptr, *biases = nullptr;   // host addresses as registered
    int bits = 0;                     // 4 = affine Q4, 8 = affine 8-bit, 16 = bf16, 40 = NVFP4
    int R = 0, C = 0;
    float stored_divisor = 0.0f, input_global_scale = 0.0f;
};

struct Seat {                         // one expert-cache seat
    int active = 0;
    int resident = 0;                 // device_address supplied by the residency arena
    uint64_t logical_id = 0;
    const uint8_t *host_base = nullptr, *payload = nullptr;
    size_t nbytes = 0;
    uint8_t *device = nullptr;        // device address of `payload`
    uint8_t *owned = nullptr;         // HBM copy made by the plain bind
    uint64_t generation = 0;
};

struct Pending { const void *staged; void *host; size_t nbytes; };

// Expert residency (include/salt/gpu_residency.h:63-89).  The ledger on the engine's side owns the protocol (which
// seat, which staging buffer, which ticket); what the backend keeps is what it needs to answer it:
//  * a staging buffer is "in flight" from populate until the copy out of it is known to be complete; it remembers the
//    ticket and the seat it feeds, and carries the one event that marks the end of its copy;
//  * a seat remembers the staging buffer that is filling it (or none);
//  * copies are spread over several streams ("lanes", staging buffer b uses lane b % lanes), so that independent fills
//    overlap on the copy engines instead of queueing behind each other.
struct Residency {
    static constexpr uint32_t kNone = 0xffffffffu;
    static constexpr int kLanes = 4;
    struct StagingBuffer {
        hipEvent_t copied = nullptr;  // recorded behind the copy out of this buffer
        uint64_t ticket = 0;          // 0: idle
        uint32_t seat = kNone;
    };
    int live = 0;                     // create succeeded and destroy has not run
    int broken = 0;                   // a copy stream failed: every later call is refused until destroy
    SaltGpuResidencyPlan plan = {};
    uint8_t *arena = nullptr, *pinned = nullptr;
    hipStream_t lanes[kLanes] = {};
    std::vector<StagingBuffer> buffers;
    std::vector<uint32_t> seat_buffer; // per seat: the staging buffer that is filling it, or kNone
    int published = 0;                // the permanent spans are populated and resolvable

    uint8_t *staging_at(uint32_t b) const { return pinned + (size_t)b * plan.staging_bytes; }
    hipStream_t lane_of(uint32_t b) const { return lanes[b % kLanes]; }
};

struct Engine {
    int mapped_only = 0, defer = 0;
    SaltGpuBatchStatsV2 stats = {};
    std::vector<Resource> resources;
    std::unordered_map<const void *, Tensor> tensors;
    std::vector<Seat> seats;
    std::vector<int> logical_seat;    // logical id -> seat or -1
    std::vector<SaltGpuSharedBuffer> shared;
    uint64_t device_copied_bytes = 0, peak_window_bytes = 0;
    // activation staging: bump regions of one pinned and one device buffer
    uint8_t *pinned = nullptr, *device = nullptr;
    uint8_t *pinned_dev = nullptr;    // the pinned region as kernels address it (zero-copy for small calls)
    size_t staging_capacity = 0, pinned_used = 0, device_used = 0;
    // scratch for weights that arrive without a resident resource
    // (chunks: a call that needs more than the current chunk holds gets another one; nothing that an earlier job of
    // the same call points at is ever moved or freed before the call ends)
    struct LegacyChunk { uint8_t *base; size_t capacity; };
    std::vector<LegacyChunk> legacy_chunks;
    size_t legacy_used = 0;           // bytes used of the last chunk
    int legacy_dirty = 0;             // some chunk holds weights of an earlier call
    int legacy_depth = 0;             // nesting of the entry points that may copy weights
    std::vector<Pending> pending;
    Residency residency;
    // component pool
    std::vector<Region> regions;      // sorted by (resource, source offset) once built
    int pool_final = 0;               // regions are resident; the set no longer grows
    uint64_t pool_bytes = 0, pool_peak_bytes = 0;
    uint64_t pool_layout_bytes = 0, pool_layout_max_span = 0;     // permanent-span layout handed to the engine
    uint32_t pool_span_count = 0;
};

Engine g_engine;

size_t align_up(size_t n, size_t a) { return (n + a - 1) / a * a; }

// ---- staging ---------------------------------------------------------------

int staging_reserve(size_t pinned_bytes, size_t device_bytes) {
    Engine &e = g_engine;
    const size_t need = align_up((pinned_bytes > device_bytes ? pinned_bytes : device_bytes) + 4096, 1 << 20);
    if (e.pinned_used + pinned_bytes <= e.staging_capacity && e.device_used + device_bytes <= e.staging_capacity)
        return 0;
    // everything staged so far must be published before the buffers move
    if (salt_gpu_sync() != 0) return -1;
    if (need <= e.staging_capacity) return 0;
    if (e.pinned) { (void)hipHostFree(e.pinned); (void)hipFree(e.device); e.pinned = e.device = nullptr; }
    e.staging_capacity = 0;
    size_t capacity = 64u << 20;
    while (capacity < need) capacity *= 2;
    if (hip_ok(hipHostMalloc((void **)&e.pinned, capacity, hipHostMallocMapped), "hipHostMalloc staging") != 0 ||
        hip_ok(hipMalloc((void **)&e.device, capacity), "hipMalloc staging") != 0)
        return -1;
    void *view = nullptr;
    e.pinned_dev = hipHostGetDevicePointer(&view, e.pinned, 0) == hipSuccess ? (uint8_t *)view : nullptr;
    (void)hipGetLastError();
    e.staging_capacity = capacity;
    return 0;
}

uint8_t *pinned_take(size_t nbytes) {
    Engine &e = g_engine;
    uint8_t *p = e.pinned + e.pinned_used;
    e.pinned_used += align_up(nbytes, 256);
    return p;
}
uint8_t *device_take(size_t nbytes) {
    Engine &e = g_engine;
    uint8_t *p = e.device + e.device_used;
    e.device_used += align_up(nbytes, 256);
    return p;
}

// Calls that return this little write their results straight into the pinned staging memory: one copy command fewer
// per call.  (Reading the activations from there as well was measured: every tile re-reads them across the bus and
// a 4096 x 4096 call went from 33 to 51 us.)
constexpr size_t ZERO_COPY_BYTES = 128 * 1024;
bool zero_copy(size_t nbytes) { return g_engine.pinned_dev != nullptr && nbytes <= ZERO_COPY_BYTES; }
uint8_t *pinned_device_view(const uint8_t *pin) { return g_engine.pinned_dev + (pin - g_engine.pinned); }

// Copies host floats to the device through pinned memory on the library stream.
float *upload_activations(const float *host, size_t count) {
    uint8_t *pin = pinned_take(count * 4), *dev = device_take(count * 4);
    memcpy(pin, host, count * 4);
    if (zero_copy(count * 4)) {
        // a few kilobytes: one small kernel reads them across the bus once (a launch costs less than a copy command)
        if (copy_words_launch(dev, pinned_device_view(pin), count, g_state.stream) != 0) {
            set_error("activation upload: copy kernel failed to launch");
            return nullptr;
        }
        return (float *)dev;
    }
    if (hip_ok(hipMemcpyAsync(dev, pin, count * 4, hipMemcpyHostToDevice, g_state.stream), "activation upload") != 0)
        return nullptr;
    return (float *)dev;
}

struct OutputCopy { uint8_t *dev; uint8_t *pin; size_t nbytes; };

// After a call has enqueued its kernels: copy every staged output back and,
// unless deferring, wait and publish.
int finish_call(const std::vector<OutputCopy> &copies) {
    for (const OutputCopy &c : copies)
        if (hip_ok(hipMemcpyAsync(c.pin, c.dev, c.nbytes, hipMemcpyDeviceToHost, g_state.stream), "output copy") != 0)
            return -1;
    if (g_engine.defer) return 0;
    return salt_gpu_sync();
}

// ---- resources ---------------------------------------------------------------

int find_resource(uint32_t kind, uint32_t id) {
    for (size_t i = 0; i < g_engine.resources.size(); ++i)
        if (g_engine.resources[i].kind == kind && g_engine.resources[i].id == id) return (int)i;
    return -1;
}

bool inside(const uint8_t *base, size_t nbytes, const void *p, size_t n) {
    const uintptr_t b = (uintptr_t)base, q = (uintptr_t)p;
    return q >= b && n <= nbytes && q - b <= nbytes - n;
}

// Device address of a host byte range that lies inside an active resource, a
// bound window or a bound expert seat; nullptr when it is not resident.
const uint8_t *resident_address(const void *host, size_t nbytes) {
    if (!host) return nullptr;
    for (const Resource &r : g_engine.resources) {
        if (!r.active) continue;
        if (r.device && inside(r.host, r.nbytes, host, nbytes)) return r.device + ((const uint8_t *)host - r.host);
        if (r.window_device && inside(r.host + r.window_offset, r.window_bytes, host, nbytes))
            return r.window_device + ((const uint8_t *)host - (r.host + r.window_offset));
    }
    for (const Region &g : g_engine.regions)
        if (g.device && inside(g.host, g.nbytes, host, nbytes)) return g.device + ((const uint8_t *)host - g.host);
    for (const Seat &s : g_engine.seats)
        if (s.active && inside(s.payload, s.nbytes - (size_t)(s.payload - s.host_base), host, nbytes))
            return s.device + ((const uint8_t *)host - s.payload);
    return nullptr;
}

int drain_device() { return hip_ok(hipDeviceSynchronize(), "hipDeviceSynchronize"); }

void forget_tensors_of(int resource_index) {
    for (auto it = g_engine.tensors.begin(); it != g_engine.tensors.end();)
        it = it->second.resource == resource_index ? g_engine.tensors.erase(it) : ++it;
}

int pool_release_resource(int resource_index);
int pool_finalize();

int release_resource_memory(Resource &r) {
    int failed = 0;
    if (r.device || r.window_device || r.pool) failed |= drain_device();      // no reader may outlive the range
    if (r.pool) failed |= pool_release_resource((int)(&r - g_engine.resources.data()));
    if (r.device) { failed |= hip_ok(hipFree(r.device), "hipFree resource"); g_engine.device_copied_bytes -= r.nbytes; }
    if (r.window_device) failed |= hip_ok(hipFree(r.window_device), "hipFree window");
    r.device = r.window_device = nullptr;
    r.window_bytes = 0;
    r.active = 0;
    return failed ? -1 : 0;
}

// ---- weights of one Q4 / NVFP4 operand -------------------------------------

struct Q4Weights { const uint8_t *vals, *scales, *biases; };

size_t q4_vals_bytes(int R, int C) { return ((size_t)R * C + 7) / 8 * 4; }
size_t q8_vals_bytes(int R, int C) { return ((size_t)R * C + 3) / 4 * 4; }
size_t q4_meta_bytes(int R, int C) { return ((size_t)R * C + 63) / 64 * 2; }

// ---- component pool -----------------------------------------------------------
//
// A resource that is pool-bound (reference gpu_hip.cpp:4208-4217) is not copied whole: only the byte ranges its
// registered tensors occupy become resident, merged into few regions.  The reference pins those host ranges; here
// they are copied to HBM, either into the residency arena as permanent spans (when the engine runs one) or into
// allocations of their own at the first salt_gpu_sync.

constexpr uint64_t POOL_GRANULE = 4096;     // a region starts on this multiple of the resource offset, so a tensor
                                            // keeps its alignment below the granule when it moves to the device
constexpr uint64_t POOL_ALIGN = 256;        // of a region inside the residency arena

void tensor_bytes(const Tensor &t, size_t *value_bytes, size_t *scale_bytes) {
    const size_t elements = (size_t)t.R * (size_t)t.C;
    if (t.bits == 4) { *value_bytes = q4_vals_bytes(t.R, t.C); *scale_bytes = q4_meta_bytes(t.R, t.C); }
    else if (t.bits == 8) { *value_bytes = q8_vals_bytes(t.R, t.C); *scale_bytes = q4_meta_bytes(t.R, t.C); }
    else if (t.bits == 16) { *value_bytes = elements * 2; *scale_bytes = 0; }
    else { *value_bytes = elements / 2; *scale_bytes = elements / 16; }
}

int pool_add_range(int ri, const uint8_t *p, size_t nbytes) {
    Engine &e = g_engine;
    const Resource &r = e.resources[(size_t)ri];
    if (!p || nbytes < 1 || !inside(r.host, r.nbytes, p, nbytes)) return -1;
    uint64_t first = (uint64_t)(p - r.host), last = first + nbytes;
    first -= first % POOL_GRANULE;
    last = (last + POOL_GRANULE - 1) / POOL_GRANULE * POOL_GRANULE;
    if (last > r.nbytes) last = r.nbytes;
    for (size_t i = 0; i < e.regions.size();) {              // merge with every range it overlaps or touches
        const Region &g = e.regions[i];
        const uint64_t g0 = g.source_offset, g1 = g0 + g.nbytes;
        if (g.resource != ri || last < g0 || g1 < first) { ++i; continue; }
        if (g0 < first) first = g0;
        if (g1 > last) last = g1;
        e.regions.erase(e.regions.begin() + (long)i);
        i = 0;
    }
    Region g;
    g.resource = ri; g.host = r.host + first; g.nbytes = (size_t)(last - first); g.source_offset = first;
    e.regions.push_back(g);
    return 0;
}

bool pool_resources_present() {
    for (const Resource &r : g_engine.resources)
        if (r.kind <= KIND_MAX && r.active && r.pool) return true;
    return false;
}

// Builds the regions from the tensors registered so far.  -1 when the pool is already resident or holds no tensor.
int pool_build_regions() {
    Engine &e = g_engine;
    if (e.pool_final) return -1;
    if (!e.regions.empty()) return 0;
    for (const auto &entry : e.tensors) {
        const Tensor &t = entry.second;
        if (t.resource < 0 || !e.resources[(size_t)t.resource].pool) continue;
        size_t vb = 0, mb = 0;
        tensor_bytes(t, &vb, &mb);
        if (pool_add_range(t.resource, t.vals, vb) != 0 || (t.scales && mb && pool_add_range(t.resource, t.scales, mb) != 0) ||
            (t.biases && mb && pool_add_range(t.resource, t.biases, mb) != 0)) {
            e.regions.clear();
            return -1;
        }
    }
    std::sort(e.regions.begin(), e.regions.end(), [](const Region &a, const Region &b) {
        return a.resource != b.resource ? a.resource < b.resource : a.source_offset < b.source_offset;
    });
    return e.regions.empty() ? -1 : 0;
}

bool pool_covers(const void *p, size_t nbytes) {
    for (const Region &g : g_engine.regions)
        if (inside(g.host, g.nbytes, p, nbytes)) return true;
    return false;
}

// Without a residency arena the regions get allocations of their own (the counterpart of the reference pinning
// them at its first sync, gpu_hip.cpp:3573-3640 and 6917-6920).  A pool that holds no tensor yet is left alone.
int pool_finalize() {
    Engine &e = g_engine;
    if (e.pool_final || !pool_resources_present()) return 0;
    if (e.pool_span_count != 0) return 0;                    // laid out as permanent spans: the engine populates them
    if (pool_build_regions() != 0) return 0;
    uint64_t total = 0;
    for (Region &g : e.regions) {
        if (hip_ok(hipMalloc((void **)&g.owned, g.nbytes), "hipMalloc component pool") != 0) { g.owned = nullptr; total = UINT64_MAX; break; }
        if (hip_ok(hipMemcpy(g.owned, g.host, g.nbytes, hipMemcpyHostToDevice), "component pool upload") != 0) { total = UINT64_MAX; break; }
        g.device = g.owned;
        total += g.nbytes;
    }
    if (total == UINT64_MAX) {
        for (Region &g : e.regions) if (g.owned) (void)hipFree(g.owned);
        e.regions.clear();
        return -1;
    }
    e.pool_bytes = total;
    if (total > e.pool_peak_bytes) e.pool_peak_bytes = total;
    e.device_copied_bytes += total;
    e.pool_final = 1;
    return 0;
}

// Drops the regions of one resource (reference gpu_hip.cpp:3642-3684); the caller has drained the device.
int pool_release_resource(int ri) {
    Engine &e = g_engine;
    int failed = 0;
    for (size_t i = 0; i < e.regions.size();) {
        Region &g = e.regions[i];
        if (g.resource != ri) { ++i; continue; }
        if (g.owned) { failed |= hip_ok(hipFree(g.owned), "hipFree component pool"); e.device_copied_bytes -= g.nbytes; }
        e.regions.erase(e.regions.begin() + (long)i);
    }
    uint64_t total = 0;
    for (const Region &g : e.regions) if (g.device) total += g.nbytes;
    e.pool_bytes = total;
    if (e.regions.empty()) e.pool_final = 0;
    e.resources[(size_t)ri].pool = 0;
    return failed ? -1 : 0;
}

// Weights that arrive outside every resident resource are copied per call.  The copies of one call stay where they
// are until the call has ended: a job enqueued early must not see a later job's weights.  The next call that copies
// weights first waits for the device (the earlier call's kernels may be deferred) and starts over.
struct LegacyScope {
    LegacyScope() {
        Engine &e = g_engine;
        if (e.legacy_depth++ == 0 && e.legacy_dirty && g_state.ready) {
            if (drain_device() == 0) {
                // keep the largest chunk, free the others
                size_t keep = 0;
                for (size_t i = 1; i < e.legacy_chunks.size(); ++i)
                    if (e.legacy_chunks[i].capacity > e.legacy_chunks[keep].capacity) keep = i;
                for (size_t i = 0; i < e.legacy_chunks.size(); ++i)
                    if (i != keep) (void)hipFree(e.legacy_chunks[i].base);
                const Engine::LegacyChunk kept = e.legacy_chunks[keep];
                e.legacy_chunks.assign(1, kept);
                e.legacy_used = 0;
                e.legacy_dirty = 0;
            }
        }
    }
    ~LegacyScope() { g_engine.legacy_depth--; }
};

int legacy_reserve(size_t nbytes) {
    Engine &e = g_engine;
    if (!e.legacy_chunks.empty() && e.legacy_used + nbytes <= e.legacy_chunks.back().capacity) return 0;
    size_t capacity = 64u << 20;
    while (capacity < nbytes) capacity *= 2;
    uint8_t *base = nullptr;
    if (hip_ok(hipMalloc((void **)&base, capacity), "hipMalloc legacy weights") != 0) return -1;
    e.legacy_chunks.push_back(Engine::LegacyChunk{base, capacity});
    e.legacy_used = 0;
    return 0;
}

const uint8_t *legacy_upload(const void *host, size_t nbytes) {
    Engine &e = g_engine;
    uint8_t *dst = e.legacy_chunks.back().base + e.legacy_used;
    e.legacy_used += align_up(nbytes, 256);
    e.legacy_dirty = 1;
    // pageable source: the runtime stages it; the copy is complete on return
    if (hip_ok(hipMemcpy(dst, host, nbytes, hipMemcpyHostToDevice), "legacy weight upload") != 0) return nullptr;
    return dst;
}

// Maps the host pointers of one affine-Q4 tensor to device addresses.
// *legacy is set when the weights had to be copied for this call.
int locate_q4(const void *vals, const void *scales, const void *biases, int R, int C, Q4Weights *out, int *legacy,
              int bits = 4) {
    const size_t vb = bits == 8 ? q8_vals_bytes(R, C) : q4_vals_bytes(R, C), mb = q4_meta_bytes(R, C);
    out->vals = resident_address(vals, vb);
    out->scales = resident_address(scales, mb);
    out->biases = biases ? resident_address(biases, mb) : nullptr;
    if (out->vals && out->scales && (!biases || out->biases)) return 0;
    if (g_engine.mapped_only) {
        g_engine.stats.mapped_only_misses++;
        set_error("weights are not inside an active resource and mapped-only mode forbids copying them");
        return -1;
    }
    if (legacy_reserve(align_up(vb, 256) + 2 * align_up(mb, 256)) != 0) return -1;
    out->vals = legacy_upload(vals, vb);
    out->scales = legacy_upload(scales, mb);
    out->biases = biases ? legacy_upload(biases, mb) : nullptr;
    if (!out->vals || !out->scales || (biases && !out->biases)) return -1;
    *legacy = 1;
    return 0;
}

// A registered key must agree with the pointers the call carries (the
// reference re-validates this on every batch, gpu_hip.cpp:4973-4986).
int key_agrees(const void *key, const void *vals, const void *scales, const void *biases, int R, int C, int bits = 4) {
    if (!key) return 1;
    auto it = g_engine.tensors.find(key);
    if (it == g_engine.tensors.end()) return 1;          // unknown keys fall through to pointer lookup
    const Tensor &t = it->second;
    return t.bits == bits && t.vals == vals && t.scales == scales && t.biases == biases && t.R == R && t.C == C;
}

void count_batch(const void *vals, int legacy) {
    SaltGpuBatchStatsV2 &s = g_engine.stats;
    if (legacy) { s.arena_batches++; return; }
    for (const Resource &r : g_engine.resources)
        if (r.active && inside(r.host, r.nbytes, vals, 1)) {
            if (r.kind == KIND_EXPERT_LAYER) s.expert_layer_batches++; else s.trunk_batches++;
            return;
        }
    s.expert_layer_batches++;                             // expert-cache seat
}

int ready_or_fail(const char *who) {
    if (g_state.ready) return 0;
    set_error("%s: salt_gpu_init has not succeeded", who);
    return -1;
}

int register_tensor(uint32_t kind, uint32_t id, const void *key, const void *vals, size_t vals_bytes,
                    const void *scales, size_t scales_bytes, const void *biases, size_t biases_bytes, Tensor proto) {
    const int ri = find_resource(kind, id);
    if (ri < 0 || !key || !vals || (!scales && scales_bytes)) { set_error("tensor slot: unknown resource or null argument"); return -1; }
    const Resource &r = g_engine.resources[(size_t)ri];
    if (!inside(r.host, r.nbytes, vals, vals_bytes) || (scales && !inside(r.host, r.nbytes, scales, scales_bytes)) ||
        (biases && !inside(r.host, r.nbytes, biases, biases_bytes))) {
        set_error("tensor slot: tensor bytes lie outside resource (%u, %u)", kind, id);
        return -1;
    }
    proto.resource = ri;
    proto.vals = (const uint8_t *)vals; proto.scales = (const uint8_t *)scales; proto.biases = (const uint8_t *)biases;
    auto it = g_engine.tensors.find(key);
    if (it != g_engine.tensors.end()) {
        const Tensor &old = it->second;
        const bool same = old.resource == ri && old.vals == proto.vals && old.scales == proto.scales &&
                          old.biases == proto.biases && old.bits == proto.bits && old.R == proto.R && old.C == proto.C;
        if (!same) { set_error("tensor slot: key is already bound to a different tensor"); return -1; }
        return 0;
    }
    if (r.pool) {
        // a pool that is laid out or resident no longer grows: the tensor must lie inside what it already holds
        size_t vb = 0, mb = 0;
        tensor_bytes(proto, &vb, &mb);
        if (g_engine.pool_final || g_engine.pool_span_count != 0) {
            if (!pool_covers(vals, vb) || (scales && mb && !pool_covers(scales, mb)) || (biases && mb && !pool_covers(biases, mb))) {
                set_error("tensor slot: the component pool of resource (%u, %u) is already laid out without these bytes", kind, id);
                return -1;
            }
        } else {
            g_engine.regions.clear();                     // rebuilt from all tensors when next needed
        }
    }
    g_engine.tensors.emplace(key, proto);
    return 0;
}

// ---- Q4 job assembly ----------------------------------------------------------

struct HostJob {                      // one matrix against `tokens` contiguous rows of x
    Q4Weights w;
    const float *x_host; float *y_host;
    const float *x_dev; float *y_dev;     // filled in when already on the device
    int rows, tokens;
};

// Runs jobs that share C.  Inputs with x_dev == nullptr are uploaded (equal
// host pointers once); outputs with y_dev == nullptr are staged for
// publication.  Token counts above four are split into groups of four.
int run_q4_jobs(std::vector<HostJob> &jobs, int C, std::vector<OutputCopy> *copies) {
    Engine &e = g_engine;
    size_t in_bytes = 0, out_bytes = 0;
    for (const HostJob &j : jobs) {
        if (!j.x_dev) in_bytes += align_up((size_t)j.tokens * C * 4, 256);
        if (!j.y_dev) out_bytes += align_up((size_t)j.tokens * j.rows * 4, 256);
    }
    if (staging_reserve(in_bytes + out_bytes, in_bytes + out_bytes) != 0) return -1;
    std::unordered_map<const float *, const float *> uploaded;
    for (HostJob &j : jobs) {
        if (!j.x_dev) {
            auto it = uploaded.find(j.x_host);
            if (it != uploaded.end()) { j.x_dev = it->second; }
            else {
                j.x_dev = upload_activations(j.x_host, (size_t)j.tokens * C);
                if (!j.x_dev) return -1;
                uploaded.emplace(j.x_host, j.x_dev);
            }
        }
        if (!j.y_dev) {
            const size_t count = (size_t)j.tokens * j.rows;
            uint8_t *dev = device_take(count * 4), *pin = pinned_take(count * 4);
            e.pending.push_back({pin, j.y_host, count * 4});
            if (zero_copy(count * 4)) {
                j.y_dev = (float *)pinned_device_view(pin);          // written in place, nothing to copy back
            } else {
                j.y_dev = (float *)dev;
                copies->push_back({dev, pin, count * 4});
            }
        }
    }
    int max_tokens = 0;
    for (const HostJob &j : jobs) max_tokens = j.tokens > max_tokens ? j.tokens : max_tokens;
    std::vector<SaltMi355Q4Job> group;
    for (int first = 0; first < max_tokens; first += 4) {
        // jobs are bucketed by how many tokens of this group of four they still have
        for (int width = 4; width >= 1; --width) {
            group.clear();
            for (const HostJob &j : jobs) {
                const int left = j.tokens - first;
                if ((left >= 4 ? 4 : left) != width) continue;
                SaltMi355Q4Job q;
                q.vals = j.w.vals; q.scales = j.w.scales; q.biases = j.w.biases;
                q.xs = j.x_dev + (size_t)first * C;
                q.ys = j.y_dev + (size_t)first * j.rows;
                q.rows = j.rows;
                group.push_back(q);
            }
            if (group.empty()) continue;
            // ys of a job is [tokens][rows]: the sub-launch writes rows `first..first+width` of it.  Bit-exact kernels
            // unless the engine has opted into the tolerance class (salt_mi355_set_tolerance_class).
            const int rc = g_state.tolerance_class
                ? salt_mi355_q4_jobs_t_dev(group.data(), (int)group.size(), C, width, g_state.stream)
                : salt_mi355_q4_jobs_dev(group.data(), (int)group.size(), C, width, 0, g_state.stream);
            if (rc != 0) return -1;
        }
    }
    return 0;
}

}  // namespace

extern "C" {

// ================================================================ lifecycle

int salt_gpu_init(void) {
    if (g_state.ready) return 0;
    if (salt_mi355_init() != 0) return -1;
    fprintf(stderr, "salt-mi355: MI355X backend ready (%d CUs, HBM-resident weights)\n", g_state.compute_units);
    return 0;
}

int salt_gpu_free(void) {
    Engine &e = g_engine;
    if (e.residency.live || e.residency.broken) { set_error("salt_gpu_free: the residency arena is still live"); return -1; }
    int failed = 0;
    if (g_state.ready) {
        failed |= salt_gpu_sync();
        failed |= drain_device();
        for (Resource &r : e.resources) failed |= release_resource_memory(r);
        for (Seat &s : e.seats) if (s.owned) failed |= hip_ok(hipFree(s.owned), "hipFree seat");
        for (SaltGpuSharedBuffer &b : e.shared) if (b.contents) failed |= hip_ok(hipHostFree(b.contents), "hipHostFree");
        if (e.pinned) { failed |= hip_ok(hipHostFree(e.pinned), "hipHostFree"); failed |= hip_ok(hipFree(e.device), "hipFree"); }
        for (const Engine::LegacyChunk &c : e.legacy_chunks) failed |= hip_ok(hipFree(c.base), "hipFree");
    }
    e = Engine();
    failed |= salt_mi355_shutdown();
    return failed ? -1 : 0;
}

int salt_gpu_cuda_present(void) { return 0; }
int salt_gpu_rocm_present(void) { return 1; }
int salt_gpu_pageable_mmap_active(void) { return 0; }
void salt_gpu_set_mapped_only(int on) { g_engine.mapped_only = on ? 1 : 0; }
int salt_gpu_mapped_only(void) { return g_engine.mapped_only; }
int salt_gpu_defer(void) { return g_engine.defer; }

int salt_gpu_set_defer(int on) {
    if (on) { g_engine.defer = 1; return 0; }
    g_engine.defer = 0;
    return salt_gpu_sync();
}

int salt_gpu_sync(void) {
    Engine &e = g_engine;
    if (!g_state.ready) return e.pending.empty() ? 0 : -1;
    if (pool_finalize() != 0) return -1;
    const int rc = hip_ok(hipStreamSynchronize(g_state.stream), "hipStreamSynchronize");
    if (rc == 0)
        for (const Pending &p : e.pending) memcpy(p.host, p.staged, p.nbytes);
    e.pending.clear();                 // after a failure nothing is published
    e.pinned_used = e.device_used = 0;
    return rc;
}

void salt_gpu_batch_stats_get(SaltGpuBatchStats *stats) {
    if (stats) memcpy(stats, &g_engine.stats, sizeof *stats);     // the V1 fields lead the V2 structure
}

int salt_gpu_batch_stats_get_v2(SaltGpuBatchStatsV2 *stats, size_t stats_size) {
    if (!stats || stats_size != sizeof *stats) return -1;
    *stats = g_engine.stats;
    return 0;
}

int salt_gpu_startup_requirements(SaltGpuStartupRequirements *req, size_t req_size) {
    if (!req || req_size != sizeof *req) return -1;
    memset(req, 0, sizeof *req);
    const uint64_t output_bytes = (uint64_t)MAX_OUTPUT_FLOATS * 4;
    const uint64_t descriptor_bytes = (uint64_t)MAX_BATCH_JOBS * sizeof(Q4Job);
    req->fixed_device_bytes = 2 * output_bytes + State::kTableSlots * descriptor_bytes;
    req->fixed_pinned_host_bytes = 2 * output_bytes + State::kTableSlots * descriptor_bytes;
    req->descriptor_bytes = 2 * descriptor_bytes;
    req->max_output_floats = MAX_OUTPUT_FLOATS;
    req->max_batch_jobs = MAX_BATCH_JOBS;
    req->shared_buffer_slots = SHARED_SLOTS;
    return 0;
}

// ================================================================ resources

int salt_gpu_weight_resource_describe(uint32_t kind, uint32_t resource_id, const void *base, size_t nbytes) {
    if (ready_or_fail("weight_resource_describe") != 0) return -1;
    if (kind > KIND_MAX || !base || nbytes < 1) { set_error("describe: bad arguments"); return -1; }
    const int ri = find_resource(kind, resource_id);
    if (ri >= 0) {
        const Resource &r = g_engine.resources[(size_t)ri];
        if (r.host == base && r.nbytes == nbytes) return 0;
        set_error("describe: resource (%u, %u) is already described differently", kind, resource_id);
        return -1;
    }
    Resource r;
    r.kind = kind; r.id = resource_id; r.host = (const uint8_t *)base; r.nbytes = nbytes;
    g_engine.resources.push_back(r);
    return 0;
}

int salt_gpu_weight_resource_activate(uint32_t kind, uint32_t resource_id, SaltGpuWeightAddressability policy) {
    if (ready_or_fail("weight_resource_activate") != 0) return -1;
    const int ri = find_resource(kind, resource_id);
    if (ri < 0) { set_error("activate: resource (%u, %u) was never described", kind, resource_id); return -1; }
    Resource &r = g_engine.resources[(size_t)ri];
    if (policy == SALT_GPU_WEIGHT_ADDRESS_PAGEABLE) {
        set_error("activate: pageable host mappings are not available on this backend");
        return -1;
    }
    if (r.active) return r.policy == (int)policy ? 0 : -1;
    if (policy == SALT_GPU_WEIGHT_ADDRESS_BOUNDED_WINDOW) {
        r.active = 1; r.policy = (int)policy;
        return 0;
    }
    if (hip_ok(hipMalloc((void **)&r.device, r.nbytes), "hipMalloc resource") != 0) { r.device = nullptr; return -1; }
    if (hip_ok(hipMemcpy(r.device, r.host, r.nbytes, hipMemcpyHostToDevice), "resource upload") != 0) {
        (void)hipFree(r.device);
        r.device = nullptr;
        return -1;
    }
    g_engine.device_copied_bytes += r.nbytes;
    r.active = 1; r.policy = (int)policy;
    return 0;
}

int salt_gpu_weight_resource_pool_bind(uint32_t kind, uint32_t resource_id) {
    if (ready_or_fail("weight_resource_pool_bind") != 0) return -1;
    const int ri = find_resource(kind, resource_id);
    if (ri < 0) { set_error("pool bind: resource (%u, %u) was never described", kind, resource_id); return -1; }
    Resource &r = g_engine.resources[(size_t)ri];
    if (!r.active || r.device || r.window_device || r.policy != SALT_GPU_WEIGHT_ADDRESS_BOUNDED_WINDOW || r.pool ||
        g_engine.pool_final || g_engine.pool_span_count != 0) {
        set_error("pool bind: the resource must be active and window-addressed with nothing bound, and the pool not yet resident");
        return -1;
    }
    r.pool = 1;
    g_engine.regions.clear();
    return 0;
}

int salt_gpu_weight_resource_deactivate(uint32_t kind, uint32_t resource_id) {
    if (ready_or_fail("weight_resource_deactivate") != 0) return -1;
    const int ri = find_resource(kind, resource_id);
    if (ri < 0) return -1;
    if (salt_gpu_sync() != 0) return -1;
    return release_resource_memory(g_engine.resources[(size_t)ri]);
}

int salt_gpu_weight_resource_bind(uint32_t kind, uint32_t resource_id, const void *base, size_t nbytes) {
    if (salt_gpu_weight_resource_describe(kind, resource_id, base, nbytes) != 0) return -1;
    return salt_gpu_weight_resource_activate(kind, resource_id, SALT_GPU_WEIGHT_ADDRESS_AUTO);
}

int salt_gpu_weight_resource_unbind(uint32_t kind, uint32_t resource_id) {
    if (ready_or_fail("weight_resource_unbind") != 0) return -1;
    const int ri = find_resource(kind, resource_id);
    if (ri < 0) return -1;
    if (salt_gpu_sync() != 0) return -1;
    const int rc = release_resource_memory(g_engine.resources[(size_t)ri]);
    forget_tensors_of(ri);
    // keep indices of the other resources stable: the record is blanked, not erased
    g_engine.resources[(size_t)ri] = Resource();
    g_engine.resources[(size_t)ri].kind = 0xFFFFFFFFu;
    return rc;
}

int salt_gpu_weight_window_bind(uint32_t kind, uint32_t resource_id, uint64_t offset, size_t nbytes) {
    if (ready_or_fail("weight_window_bind") != 0) return -1;
    const int ri = find_resource(kind, resource_id);
    if (ri < 0) return -1;
    Resource &r = g_engine.resources[(size_t)ri];
    if (!r.active || r.policy != SALT_GPU_WEIGHT_ADDRESS_BOUNDED_WINDOW || r.window_device || r.pool || nbytes < 1 ||
        offset > r.nbytes || nbytes > r.nbytes - offset) {
        set_error("window bind: resource is not window-addressed, is pool-bound, a window is already bound, or the range is bad");
        return -1;
    }
    if (hip_ok(hipMalloc((void **)&r.window_device, nbytes), "hipMalloc window") != 0) { r.window_device = nullptr; return -1; }
    if (hip_ok(hipMemcpy(r.window_device, r.host + offset, nbytes, hipMemcpyHostToDevice), "window upload") != 0) {
        (void)hipFree(r.window_device);
        r.window_device = nullptr;
        return -1;
    }
    r.window_offset = offset; r.window_bytes = nbytes;
    if (nbytes > g_engine.peak_window_bytes) g_engine.peak_window_bytes = nbytes;
    return 0;
}

int salt_gpu_weight_window_unbind(uint32_t kind, uint32_t resource_id) {
    if (ready_or_fail("weight_window_unbind") != 0) return -1;
    const int ri = find_resource(kind, resource_id);
    if (ri < 0) return -1;
    Resource &r = g_engine.resources[(size_t)ri];
    if (!r.window_device) return 0;
    if (salt_gpu_sync() != 0 || drain_device() != 0) return -1;
    const int rc = hip_ok(hipFree(r.window_device), "hipFree window");
    r.window_device = nullptr; r.window_bytes = 0;
    return rc;
}

int salt_gpu_weight_resource_usage(SaltGpuWeightResourceUsage *usage, size_t usage_size) {
    if (!usage || usage_size != sizeof *usage) return -1;
    memset(usage, 0, sizeof *usage);
    for (const Resource &r : g_engine.resources) {
        if (r.kind > KIND_MAX) continue;
        usage->described_bytes += r.nbytes;
        usage->described_resources++;
        if (!r.active) continue;
        usage->active_resources++;
        if (r.device) usage->registered_bytes += r.nbytes;
        if (r.window_device) { usage->active_window_bytes += r.window_bytes; usage->active_windows++; }
        if (r.pool) usage->active_windows++;              // reference gpu_hip.cpp:4258-4272
    }
    usage->peak_window_bytes = g_engine.peak_window_bytes > g_engine.pool_peak_bytes ? g_engine.peak_window_bytes
                                                                                     : g_engine.pool_peak_bytes;
    usage->device_copied_weight_bytes = g_engine.device_copied_bytes;
    if (g_engine.residency.published) usage->device_copied_weight_bytes += g_engine.pool_bytes;
    else usage->active_window_bytes += g_engine.pool_bytes;
    return 0;
}

int salt_gpu_weight_resource_slot(uint32_t kind, uint32_t resource_id, const void *key, const uint32_t *vals,
                                  const uint16_t *scales, const uint16_t *biases, int bits, int R, int C) {
    if (ready_or_fail("weight_resource_slot") != 0) return -1;
    if (bits != 4 && bits != 8) { set_error("weight_resource_slot: only 4-bit and 8-bit tensors are on this backend's path (bits %d)", bits); return -1; }
    if (R < 1 || C < 1 || C > MAX_C) { set_error("weight_resource_slot: bad geometry"); return -1; }
    Tensor t;
    t.bits = bits; t.R = R; t.C = C;
    return register_tensor(kind, resource_id, key, vals, bits == 8 ? q8_vals_bytes(R, C) : q4_vals_bytes(R, C), scales,
                           q4_meta_bytes(R, C), biases, q4_meta_bytes(R, C), t);
}

int salt_gpu_nvfp4_resource_slot(uint32_t kind, uint32_t resource_id, const void *key, const uint8_t *packed,
                                 const uint8_t *scales, const float *weight_global_scale,
                                 const float *input_global_scale, int R, int C) {
    if (ready_or_fail("nvfp4_resource_slot") != 0) return -1;
    if (!weight_global_scale || !input_global_scale || R < 1 || C < 32 || (C & 31) || C > MAX_C ||
        !isfinite(*weight_global_scale) || *weight_global_scale == 0.0f || !isfinite(*input_global_scale) ||
        *input_global_scale <= 0.0f) {
        set_error("nvfp4_resource_slot: bad geometry or global scales");
        return -1;
    }
    Tensor t;
    t.bits = 40; t.R = R; t.C = C;
    t.stored_divisor = *weight_global_scale; t.input_global_scale = *input_global_scale;
    return register_tensor(kind, resource_id, key, packed, (size_t)R * C / 2, scales, (size_t)R * C / 16, nullptr, 0, t);
}

int salt_gpu_expert_resource_bind(uint32_t resource_id, const void *base, size_t nbytes) {
    return salt_gpu_weight_resource_bind(KIND_EXPERT_LAYER, resource_id, base, nbytes);
}
int salt_gpu_expert_resource_slot(uint32_t resource_id, const void *key, const uint32_t *vals,
                                  const uint16_t *scales, const uint16_t *biases, int R, int C) {
    return salt_gpu_weight_resource_slot(KIND_EXPERT_LAYER, resource_id, key, vals, scales, biases, 4, R, C);
}
int salt_gpu_expert_resource_unbind(uint32_t resource_id) {
    return salt_gpu_weight_resource_unbind(KIND_EXPERT_LAYER, resource_id);
}

int salt_gpu_resident_slot(const void *key, const uint32_t *vals, const uint16_t *scales, const uint16_t *biases,
                           int R, int C) {
    if (ready_or_fail("resident_slot") != 0) return -1;
    for (const Resource &r : g_engine.resources)
        if (r.active && r.kind == KIND_EXPERT_LAYER && inside(r.host, r.nbytes, vals, 1))
            return salt_gpu_weight_resource_slot(r.kind, r.id, key, vals, scales, biases, 4, R, C);
    return -1;
}

// ================================================================ shared buffers

int salt_gpu_shared_buffer_alloc(SaltGpuSharedBuffer *buffer, size_t nbytes) {
    if (!buffer) return -1;
    memset(buffer, 0, sizeof *buffer);
    if (ready_or_fail("shared_buffer_alloc") != 0 || nbytes < 1) return -1;
    void *host = nullptr, *dev = nullptr;
    if (hip_ok(hipHostMalloc(&host, nbytes, hipHostMallocMapped), "hipHostMalloc shared buffer") != 0) return -1;
    if (hip_ok(hipHostGetDevicePointer(&dev, host, 0), "hipHostGetDevicePointer") != 0 || !dev) {
        (void)hipHostFree(host);
        return -1;
    }
    memset(host, 0, nbytes);
    buffer->contents = host; buffer->nbytes = nbytes; buffer->backend = dev;
    g_engine.shared.push_back(*buffer);
    return 0;
}

int salt_gpu_shared_buffer_free(SaltGpuSharedBuffer *buffer) {
    if (!buffer) return -1;
    int rc = 0;
    if (buffer->contents) {
        if (g_state.ready && (salt_gpu_sync() != 0 || drain_device() != 0)) return -1;
        for (size_t i = 0; i < g_engine.shared.size(); ++i)
            if (g_engine.shared[i].contents == buffer->contents) {
                g_engine.shared.erase(g_engine.shared.begin() + (long)i);
                rc = hip_ok(hipHostFree(buffer->contents), "hipHostFree shared buffer");
                break;
            }
    }
    memset(buffer, 0, sizeof *buffer);
    return rc;
}

}  // extern "C"

namespace {

// Device view of a host range inside a shared buffer, or nullptr.
void *shared_device_view(const void *host, size_t nbytes) {
    for (const SaltGpuSharedBuffer &b : g_engine.shared)
        if (inside((const uint8_t *)b.contents, b.nbytes, host, nbytes))
            return (uint8_t *)b.backend + ((const uint8_t *)host - (const uint8_t *)b.contents);
    return nullptr;
}

}  // namespace

extern "C" {

// ================================================================ affine Q4

int salt_gpu_q4_matvec(const uint32_t *vals, const uint16_t *scales, const uint16_t *biases, int R, int C,
                       const float *x, float *y) {
    LegacyScope weights_of_this_call;
    if (ready_or_fail("q4_matvec") != 0) return -1;
    if (!vals || !scales || !x || !y || R < 1 || C < 1 || C > MAX_C || (size_t)R > MAX_OUTPUT_FLOATS) {
        set_error("q4_matvec: bad arguments");
        return -1;
    }
    HostJob job = {};
    int legacy = 0;
    if (locate_q4(vals, scales, biases, R, C, &job.w, &legacy) != 0) return -1;
    job.x_host = x; job.y_host = y; job.rows = R; job.tokens = 1;
    std::vector<HostJob> jobs(1, job);
    std::vector<OutputCopy> copies;
    if (run_q4_jobs(jobs, C, &copies) != 0) { (void)salt_gpu_sync(); return -1; }
    count_batch(vals, legacy);
    return finish_call(copies);
}

int salt_gpu_q4_batch(const uint32_t *const *vals, const uint16_t *const *scales, const uint16_t *const *biases,
                      const float *const *xs, float *const *ys, const void *const *ids, const int *Rj, int C,
                      int njobs) {
    LegacyScope weights_of_this_call;
    if (ready_or_fail("q4_batch") != 0) return -1;
    if (!vals || !scales || !xs || !ys || !Rj || njobs < 1 || (uint32_t)njobs > MAX_BATCH_JOBS || C < 1 || C > MAX_C) {
        set_error("q4_batch: bad arguments");
        return -1;
    }
    std::vector<HostJob> jobs;
    int any_legacy = 0;
    for (int j = 0; j < njobs; ++j) {
        const uint16_t *bias = biases ? biases[j] : nullptr;
        if (!vals[j] || !scales[j] || !xs[j] || !ys[j] || Rj[j] < 1) { set_error("q4_batch: job %d is malformed", j); return -1; }
        if (!key_agrees(ids ? ids[j] : nullptr, vals[j], scales[j], bias, Rj[j], C)) {
            set_error("q4_batch: job %d does not match the tensor registered under its key", j);
            return -1;
        }
        // consecutive jobs on the same weight with contiguous x / y become tokens of one job
        if (!jobs.empty()) {
            HostJob &prev = jobs.back();
            if (prev.rows == Rj[j] && prev.x_host + (size_t)prev.tokens * C == xs[j] &&
                prev.y_host + (size_t)prev.tokens * prev.rows == ys[j] &&
                prev.w.vals == resident_address(vals[j], 1)) {
                prev.tokens++;
                continue;
            }
        }
        HostJob job = {};
        int legacy = 0;
        if (locate_q4(vals[j], scales[j], bias, Rj[j], C, &job.w, &legacy) != 0) return -1;
        any_legacy |= legacy;
        job.x_host = xs[j]; job.y_host = ys[j]; job.rows = Rj[j]; job.tokens = 1;
        jobs.push_back(job);
    }
    std::vector<OutputCopy> copies;
    if (run_q4_jobs(jobs, C, &copies) != 0) { (void)salt_gpu_sync(); return -1; }
    count_batch(vals[0], any_legacy);
    return finish_call(copies);
}

int salt_gpu_proj_batch(const uint32_t *vals, const uint16_t *scales, const uint16_t *biases, int R, int C, int B,
                        const float *const *xs, float *const *ys, const void *id) {
    LegacyScope weights_of_this_call;
    if (ready_or_fail("proj_batch") != 0) return -1;
    if (!vals || !scales || !xs || !ys || R < 1 || C < 1 || C > MAX_C || B < 1 || B > MAX_PROJ_BATCH ||
        (uint64_t)B * (uint64_t)R > MAX_OUTPUT_FLOATS) {
        set_error("proj_batch: bad arguments");
        return -1;
    }
    for (int b = 0; b < B; ++b)                      // the reference requires one contiguous [B][C] / [B][R] pair
        if (xs[b] != xs[0] + (size_t)b * C || ys[b] != ys[0] + (size_t)b * R) {
            set_error("proj_batch: tokens are not contiguous");
            return -1;
        }
    if (!key_agrees(id, vals, scales, biases, R, C)) { set_error("proj_batch: key mismatch"); return -1; }
    HostJob job = {};
    int legacy = 0;
    if (locate_q4(vals, scales, biases, R, C, &job.w, &legacy) != 0) return -1;
    job.x_host = xs[0]; job.y_host = ys[0]; job.rows = R; job.tokens = B;
    std::vector<HostJob> jobs(1, job);
    std::vector<OutputCopy> copies;
    if (run_q4_jobs(jobs, C, &copies) != 0) { (void)salt_gpu_sync(); return -1; }
    count_batch(vals, legacy);
    if (B > 1) g_engine.stats.q4_weight_stationary_batches++;
    return finish_call(copies);
}

int salt_gpu_proj_batch_indexed(const uint32_t *vals, const uint16_t *scales, const uint16_t *biases, int R, int C,
                                int B, int first_job, int job_count, const float *xs, SaltGpuSharedBuffer *output,
                                size_t y_float_offset, const void *id) {
    LegacyScope weights_of_this_call;
    if (ready_or_fail("proj_batch_indexed") != 0) return -1;
    if (!vals || !scales || !xs || !output || !output->contents || R < 1 || C < 1 || C > MAX_C || B < 2 ||
        B > MAX_PROJ_BATCH || first_job < 0 || job_count < 1 || first_job > B - job_count) {
        set_error("proj_batch_indexed: bad arguments");
        return -1;
    }
    const size_t end = y_float_offset + (size_t)B * R;
    if (end < y_float_offset || end > output->nbytes / 4 ||
        !shared_device_view(output->contents, output->nbytes)) {
        set_error("proj_batch_indexed: output range is not inside a shared buffer");
        return -1;
    }
    if (!key_agrees(id, vals, scales, biases, R, C)) { set_error("proj_batch_indexed: key mismatch"); return -1; }
    HostJob job = {};
    int legacy = 0;
    if (locate_q4(vals, scales, biases, R, C, &job.w, &legacy) != 0) return -1;
    job.x_host = xs + (size_t)first_job * C;
    job.y_dev = (float *)output->backend + y_float_offset + (size_t)first_job * R;   // written in place
    job.rows = R; job.tokens = job_count;
    std::vector<HostJob> jobs(1, job);
    std::vector<OutputCopy> copies;
    if (run_q4_jobs(jobs, C, &copies) != 0) { (void)salt_gpu_sync(); return -1; }
    count_batch(vals, legacy);
    g_engine.stats.direct_output_batches++;
    g_engine.stats.direct_output_jobs += (uint64_t)job_count;
    return 0;                                        // publication is salt_gpu_sync()
}

int salt_gpu_proj_batch_indexed_exact_views(const uint32_t *vals, const uint16_t *scales, const uint16_t *biases,
                                            int R, int C, int B, int first_job, int job_count, const float *xs,
                                            SaltGpuSharedBuffer *output, size_t y_float_offset, const void *id) {
    return salt_gpu_proj_batch_indexed(vals, scales, biases, R, C, B, first_job, job_count, xs, output, y_float_offset,
                                       id);
}

}  // extern "C"

namespace {

// gate, up, gelu*up, down for `count` experts whose rows are grouped in order.
// `seats_only` makes every expert resolve through its bound cache seat.
int moe_chain(const SaltGpuMoeExpert *experts, int count, int hidden, int routed, const float *inputs,
              float *outputs, float *gate_scratch, float *up_scratch, size_t scratch_capacity, int seats_only) {
    LegacyScope weights_of_this_call;
    if (ready_or_fail("q4_moe_chain") != 0) return -1;
    if (!experts || !inputs || !outputs || !gate_scratch || !up_scratch || scratch_capacity < 1 || count < 1 ||
        count > 128 || hidden < 1 || routed < 1 || hidden > MAX_C || routed > MAX_C) {
        set_error("q4_moe_chain: bad arguments");
        return -1;
    }
    uint64_t rows = 0;
    for (int i = 0; i < count; ++i) {
        if (experts[i].group < 1) { set_error("q4_moe_chain: expert %d has no rows", i); return -1; }
        rows += (uint64_t)experts[i].group;
    }
    if (rows * (uint64_t)hidden > MAX_OUTPUT_FLOATS || rows * (uint64_t)routed * 2 > MAX_OUTPUT_FLOATS ||
        rows * (uint64_t)routed > scratch_capacity) {
        set_error("q4_moe_chain: %llu rows exceed the output or scratch capacity", (unsigned long long)rows);
        return -1;
    }
    Engine &e = g_engine;
    std::vector<Q4Weights> gate((size_t)count), up((size_t)count), down((size_t)count);
    int any_legacy = 0;
    for (int i = 0; i < count; ++i) {
        const SaltGpuMoeExpert &x = experts[i];
        if (seats_only) {
            if (x.resource_slot < 0 || (size_t)x.resource_slot >= e.seats.size() ||
                !e.seats[(size_t)x.resource_slot].active ||
                e.seats[(size_t)x.resource_slot].logical_id != x.logical_resource_id) {
                set_error("q4_moe_chain_selected: expert %d is not the resource bound to seat %d", i, x.resource_slot);
                return -1;
            }
        }
        if (!key_agrees(x.gate_id, x.gate_vals, x.gate_scales, x.gate_biases, routed, hidden) ||
            !key_agrees(x.up_id, x.up_vals, x.up_scales, x.up_biases, routed, hidden) ||
            !key_agrees(x.down_id, x.down_vals, x.down_scales, x.down_biases, hidden, routed)) {
            set_error("q4_moe_chain: expert %d does not match its registered tensors", i);
            return -1;
        }
        int legacy = 0;
        if (locate_q4(x.gate_vals, x.gate_scales, x.gate_biases, routed, hidden, &gate[(size_t)i], &legacy) != 0 ||
            locate_q4(x.up_vals, x.up_scales, x.up_biases, routed, hidden, &up[(size_t)i], &legacy) != 0 ||
            locate_q4(x.down_vals, x.down_scales, x.down_biases, hidden, routed, &down[(size_t)i], &legacy) != 0)
            return -1;
        any_legacy |= legacy;
    }
    const size_t in_floats = (size_t)rows * hidden, mid_floats = (size_t)rows * routed;
    const size_t dev_bytes = align_up(in_floats * 4, 256) * 2 + align_up(mid_floats * 4, 256) * 3;
    if (staging_reserve(align_up(in_floats * 4, 256) * 2, dev_bytes) != 0) return -1;
    // Activations that already sit in a shared buffer (pinned, with a device view: the selected chain's contract) skip
    // the host copies through the staging memory: the device copies the inputs straight out of the buffer, and small
    // results are written through the buffer's device view, so that nothing is left to publish.
    const uint8_t *in_view = seats_only ? (const uint8_t *)shared_device_view(inputs, in_floats * 4) : nullptr;
    uint8_t *out_view = seats_only ? (uint8_t *)shared_device_view(outputs, in_floats * 4) : nullptr;
    const float *x_dev;
    if (in_view) {
        uint8_t *dev = device_take(in_floats * 4);
        if (hip_ok(hipMemcpyAsync(dev, inputs, in_floats * 4, hipMemcpyHostToDevice, g_state.stream), "activation upload") != 0)
            return -1;
        x_dev = (const float *)dev;
    } else {
        x_dev = upload_activations(inputs, in_floats);
    }
    if (!x_dev) return -1;
    float *gate_dev = (float *)device_take(mid_floats * 4), *up_dev = (float *)device_take(mid_floats * 4);
    float *act_dev = (float *)device_take(mid_floats * 4);
    uint8_t *out_dev = device_take(in_floats * 4), *out_pin = pinned_take(in_floats * 4);
    const bool out_direct = out_view != nullptr && zero_copy(in_floats * 4);
    const bool out_in_place = out_direct || zero_copy(in_floats * 4);
    if (out_direct) out_dev = out_view;
    else if (out_in_place) out_dev = pinned_device_view(out_pin);
    std::vector<HostJob> jobs;
    size_t row = 0;
    for (int i = 0; i < count; ++i) {
        const int g = experts[i].group;
        HostJob a = {}, b = {};
        a.w = gate[(size_t)i]; a.x_dev = x_dev + row * hidden; a.y_dev = gate_dev + row * routed; a.rows = routed; a.tokens = g;
        b.w = up[(size_t)i];   b.x_dev = x_dev + row * hidden; b.y_dev = up_dev + row * routed;   b.rows = routed; b.tokens = g;
        jobs.push_back(a); jobs.push_back(b);
        row += (size_t)g;
    }
    std::vector<OutputCopy> none;
    if (run_q4_jobs(jobs, hidden, &none) != 0) { (void)salt_gpu_sync(); return -1; }
    // Decode shape (one row per expert): gelu_tanh(gate) * up is computed in the prologue of the down launch.
    // (the tolerance-class kernels take the activation as a vector: that policy keeps the activation launch)
    bool one_row_each = !g_state.tolerance_class && (routed & 63) == 0 && routed <= 4096;
    for (int i = 0; i < count && one_row_each; ++i)
        one_row_each = experts[i].group == 1 && ((uintptr_t)down[(size_t)i].vals & 3) == 0 &&
                       ((uintptr_t)down[(size_t)i].scales & 1) == 0 && ((uintptr_t)down[(size_t)i].biases & 1) == 0;
    if (one_row_each) {
        std::vector<SaltMi355Q4Job> activated((size_t)count);
        for (int i = 0; i < count; ++i) {
            SaltMi355Q4Job &q = activated[(size_t)i];
            q.vals = down[(size_t)i].vals; q.scales = down[(size_t)i].scales; q.biases = down[(size_t)i].biases;
            q.xs = gate_dev + (size_t)i * routed;
            q.ys = (float *)out_dev + (size_t)i * hidden;
            q.rows = hidden;
        }
        if (salt_mi355_q4_jobs_activated_dev(activated.data(), count, routed, (long long)(up_dev - gate_dev), g_state.stream) != 0) {
            (void)salt_gpu_sync();
            return -1;
        }
        if (!out_direct) e.pending.push_back({out_pin, outputs, in_floats * 4});
        std::vector<OutputCopy> copies;
        if (!out_in_place) copies.push_back(OutputCopy{out_dev, out_pin, in_floats * 4});
        count_batch(experts[0].gate_vals, any_legacy);
        return finish_call(copies);
    }
    if (salt_mi355_moe_activate_dev(gate_dev, up_dev, act_dev, mid_floats, g_state.stream) != 0) { (void)salt_gpu_sync(); return -1; }
    jobs.clear();
    row = 0;
    for (int i = 0; i < count; ++i) {
        const int g = experts[i].group;
        HostJob d = {};
        d.w = down[(size_t)i]; d.x_dev = act_dev + row * routed; d.y_dev = (float *)out_dev + row * hidden; d.rows = hidden; d.tokens = g;
        jobs.push_back(d);
        row += (size_t)g;
    }
    if (run_q4_jobs(jobs, routed, &none) != 0) { (void)salt_gpu_sync(); return -1; }
    if (!out_direct) e.pending.push_back({out_pin, outputs, in_floats * 4});
    std::vector<OutputCopy> copies;
    if (!out_in_place) copies.push_back(OutputCopy{out_dev, out_pin, in_floats * 4});
    count_batch(experts[0].gate_vals, any_legacy);
    return finish_call(copies);
}

}  // namespace

extern "C" {

int salt_gpu_q4_moe_chain(const SaltGpuMoeExpert *experts, int count, int hidden, int routed, const float *inputs,
                          float *outputs, float *gate_scratch, float *up_scratch, size_t scratch_float_capacity) {
    return moe_chain(experts, count, hidden, routed, inputs, outputs, gate_scratch, up_scratch,
                     scratch_float_capacity, 0);
}

int salt_gpu_q4_moe_chain_selected(const SaltGpuMoeExpert *experts, int count, int hidden, int routed,
                                   const float *inputs, float *outputs, float *gate_scratch, float *up_scratch,
                                   size_t scratch_float_capacity) {
    // the four activation buffers must be shared buffers (reference gpu_hip.cpp:6214-6233)
    size_t rows = 0;
    for (int i = 0; experts && i < count; ++i) rows += experts[i].group > 0 ? (size_t)experts[i].group : 0;
    if (!inputs || !outputs || !gate_scratch || !up_scratch || rows < 1 ||
        !shared_device_view(inputs, rows * (size_t)hidden * 4) || !shared_device_view(outputs, rows * (size_t)hidden * 4) ||
        !shared_device_view(gate_scratch, 4) || !shared_device_view(up_scratch, 4)) {
        set_error("q4_moe_chain_selected: inputs, outputs and scratch must lie in shared buffers");
        return -1;
    }
    return moe_chain(experts, count, hidden, routed, inputs, outputs, gate_scratch, up_scratch,
                     scratch_float_capacity, 1);
}

int salt_gpu_q4_selected_shared(const SaltGpuSelectedProjectionJob *jobs, int job_count, SaltGpuSharedBuffer *arena) {
    LegacyScope weights_of_this_call;
    if (ready_or_fail("q4_selected_shared") != 0) return -1;
    if (!jobs || job_count < 1 || job_count > 256 || !arena || !arena->contents ||
        !shared_device_view(arena->contents, arena->nbytes)) {
        set_error("q4_selected_shared: bad arguments");
        return -1;
    }
    struct Range { uintptr_t lo, hi; };
    std::vector<Range> ranges;
    std::unordered_map<int, std::vector<HostJob>> by_cols;
    for (int j = 0; j < job_count; ++j) {
        const SaltGpuSelectedProjectionJob &s = jobs[j];
        if (!s.vals || !s.scales || !s.inputs || !s.outputs || s.rows < 1 || s.cols < 1 || s.cols > MAX_C || s.batch < 1 ||
            ((uintptr_t)s.inputs & 3) || ((uintptr_t)s.outputs & 3) ||
            !inside((const uint8_t *)arena->contents, arena->nbytes, s.inputs, (size_t)s.batch * s.cols * 4) ||
            !inside((const uint8_t *)arena->contents, arena->nbytes, s.outputs, (size_t)s.batch * s.rows * 4)) {
            set_error("q4_selected_shared: job %d lies outside the arena or is malformed", j);
            return -1;
        }
        const Range out = {(uintptr_t)s.outputs, (uintptr_t)s.outputs + (size_t)s.batch * s.rows * 4};
        const Range in = {(uintptr_t)s.inputs, (uintptr_t)s.inputs + (size_t)s.batch * s.cols * 4};
        if (out.lo < in.hi && in.lo < out.hi) { set_error("q4_selected_shared: job %d overlaps itself", j); return -1; }
        for (const Range &r : ranges)
            if (out.lo < r.hi && r.lo < out.hi) { set_error("q4_selected_shared: outputs overlap"); return -1; }
        ranges.push_back(out);
        if (s.resource_slot >= 0 && ((size_t)s.resource_slot >= g_engine.seats.size() ||
                                     !g_engine.seats[(size_t)s.resource_slot].active ||
                                     g_engine.seats[(size_t)s.resource_slot].logical_id != s.logical_resource_id)) {
            set_error("q4_selected_shared: job %d names a seat that holds another resource", j);
            return -1;
        }
        HostJob h = {};
        int legacy = 0;
        if (locate_q4(s.vals, s.scales, s.biases, s.rows, s.cols, &h.w, &legacy) != 0) return -1;
        h.x_host = s.inputs;                         // uploaded from the arena: inputs may be rewritten by the host later
        h.y_dev = (float *)shared_device_view(s.outputs, 4);
        h.rows = s.rows; h.tokens = s.batch;
        by_cols[s.cols].push_back(h);
    }
    std::vector<OutputCopy> none;
    for (auto &entry : by_cols)
        if (run_q4_jobs(entry.second, entry.first, &none) != 0) { (void)salt_gpu_sync(); return -1; }
    g_engine.stats.expert_layer_batches++;
    return salt_gpu_sync();                          // synchronous by contract
}

// ================================================================ expert-cache seats

int salt_gpu_selected_resources_prepare(int capacity, int logical_capacity) {
    if (ready_or_fail("selected_resources_prepare") != 0) return -1;
    if (capacity < 1 || logical_capacity < 1 || capacity > (1 << 20) || logical_capacity > (1 << 24)) return -1;
    Engine &e = g_engine;
    if (!e.seats.empty())
        return ((int)e.seats.size() == capacity && (int)e.logical_seat.size() == logical_capacity) ? 0 : -1;
    e.seats.assign((size_t)capacity, Seat());
    e.logical_seat.assign((size_t)logical_capacity, -1);
    return 0;
}

static int seat_checks(int slot, uint64_t logical_id) {
    Engine &e = g_engine;
    if (e.seats.empty() || slot < 0 || (size_t)slot >= e.seats.size() || logical_id >= e.logical_seat.size()) {
        set_error("selected resource: seat %d or logical id %llu out of range", slot, (unsigned long long)logical_id);
        return -1;
    }
    return 0;
}

int salt_gpu_selected_resource_bind(int slot, uint64_t logical_id, const void *base, size_t nbytes,
                                    const void *payload) {
    if (ready_or_fail("selected_resource_bind") != 0 || seat_checks(slot, logical_id) != 0) return -1;
    if (!base || !payload || nbytes < 1 || !inside((const uint8_t *)base, nbytes, payload, 1)) return -1;
    Engine &e = g_engine;
    Seat &s = e.seats[(size_t)slot];
    if (s.active)          // an identical bind is an idempotent reuse (reference gpu_hip.cpp:6516-6527)
        return (!s.resident && s.logical_id == logical_id && s.host_base == base && s.payload == payload &&
                s.nbytes == nbytes) ? 0 : -1;
    if (e.logical_seat[(size_t)logical_id] != -1) return -1;
    uint8_t *dev = nullptr;
    if (hip_ok(hipMalloc((void **)&dev, nbytes), "hipMalloc seat") != 0) return -1;
    if (hip_ok(hipMemcpy(dev, base, nbytes, hipMemcpyHostToDevice), "seat upload") != 0) { (void)hipFree(dev); return -1; }
    s = Seat();
    s.active = 1; s.logical_id = logical_id; s.host_base = (const uint8_t *)base; s.payload = (const uint8_t *)payload;
    s.nbytes = nbytes; s.owned = dev; s.device = dev + ((const uint8_t *)payload - (const uint8_t *)base);
    e.logical_seat[(size_t)logical_id] = slot;
    e.device_copied_bytes += nbytes;
    return 0;
}

int salt_gpu_selected_resource_bind_resident(int slot, uint64_t logical_id, const void *payload, size_t nbytes,
                                             uintptr_t device_address, uint64_t generation) {
    if (ready_or_fail("selected_resource_bind_resident") != 0 || seat_checks(slot, logical_id) != 0) return -1;
    Engine &e = g_engine;
    const Residency &res = e.residency;
    if (!payload || nbytes < 1 || !device_address || !res.live || res.broken ||
        device_address < (uintptr_t)res.arena || nbytes > res.plan.device_budget_bytes ||
        device_address - (uintptr_t)res.arena > res.plan.device_budget_bytes - nbytes) {
        set_error("bind_resident: the device address is not inside the residency arena");
        return -1;
    }
    Seat &s = e.seats[(size_t)slot];
    if (s.active)
        return (s.resident && s.logical_id == logical_id && s.payload == payload && s.nbytes == nbytes &&
                s.device == (uint8_t *)device_address && s.generation == generation) ? 0 : -1;
    if (e.logical_seat[(size_t)logical_id] != -1) return -1;
    s = Seat();
    s.active = 1; s.resident = 1; s.logical_id = logical_id;
    s.host_base = s.payload = (const uint8_t *)payload; s.nbytes = nbytes;
    s.device = (uint8_t *)device_address; s.generation = generation;
    e.logical_seat[(size_t)logical_id] = slot;
    return 0;
}

int salt_gpu_selected_resources_fence(void) {
    if (ready_or_fail("selected_resources_fence") != 0) return -1;
    if (salt_gpu_sync() != 0) return -1;
    return drain_device();
}

int salt_gpu_selected_resource_unbind(int slot, uint64_t logical_id) {
    if (ready_or_fail("selected_resource_unbind") != 0 || seat_checks(slot, logical_id) != 0) return -1;
    Engine &e = g_engine;
    Seat &s = e.seats[(size_t)slot];
    if (!s.active) return 0;                              // reference gpu_hip.cpp:6637
    if (s.logical_id != logical_id) return -1;
    if (salt_gpu_selected_resources_fence() != 0) return -1;
    int rc = 0;
    if (s.owned) { rc = hip_ok(hipFree(s.owned), "hipFree seat"); e.device_copied_bytes -= s.nbytes; }
    e.logical_seat[(size_t)logical_id] = -1;
    s = Seat();
    return rc;
}

// ================================================================ NVFP4

int salt_gpu_nvfp4_qdq(const float *input, int C, float input_global_scale, uint8_t *packed, uint8_t *scales,
                       float *dequant) {
    if (ready_or_fail("nvfp4_qdq") != 0) return -1;
    if (!input || !packed || !scales || !dequant || C < 16 || (C & 15) || C > MAX_C || !isfinite(input_global_scale) ||
        input_global_scale <= 0.0f) {
        set_error("nvfp4_qdq: bad arguments");
        return -1;
    }
    if (salt_gpu_sync() != 0) return -1;                  // the status word below needs a quiet stream
    const size_t n = (size_t)C;
    if (staging_reserve(n * 10 + 4096, n * 10 + 4096) != 0) return -1;
    float *x_dev = upload_activations(input, n);
    if (!x_dev) return -1;
    uint8_t *dq_dev = device_take(n * 4), *p_dev = device_take(n / 2), *s_dev = device_take(n / 16);
    int *st_dev = (int *)device_take(4);
    uint8_t *pin = pinned_take(n * 4 + n / 2 + n / 16 + 64);
    if (clear_words_launch(st_dev, 1, g_state.stream) != 0 ||
        salt_mi355_nvfp4_qdq_dev(x_dev, C, 1, input_global_scale, p_dev, s_dev, (float *)dq_dev, st_dev, g_state.stream) != 0)
        return -1;
    int status = 0;
    uint8_t *pin_p = pin + n * 4, *pin_s = pin_p + n / 2;
    if (hip_ok(hipMemcpyAsync(pin, dq_dev, n * 4, hipMemcpyDeviceToHost, g_state.stream), "qdq copy") != 0 ||
        hip_ok(hipMemcpyAsync(pin_p, p_dev, n / 2, hipMemcpyDeviceToHost, g_state.stream), "qdq copy") != 0 ||
        hip_ok(hipMemcpyAsync(pin_s, s_dev, n / 16, hipMemcpyDeviceToHost, g_state.stream), "qdq copy") != 0 ||
        hip_ok(hipMemcpyAsync(pin_s + align_up(n / 16, 4), st_dev, 4, hipMemcpyDeviceToHost, g_state.stream), "qdq copy") != 0 ||
        hip_ok(hipStreamSynchronize(g_state.stream), "qdq sync") != 0) {
        (void)salt_gpu_sync();
        return -1;
    }
    memcpy(&status, pin_s + align_up(n / 16, 4), 4);
    g_engine.pinned_used = g_engine.device_used = 0;
    if (status != 0) { set_error("nvfp4_qdq: the activation holds a non-finite value"); return -1; }
    memcpy(dequant, pin, n * 4);
    memcpy(packed, pin_p, n / 2);
    memcpy(scales, pin_s, n / 16);
    return 0;
}

}  // extern "C"

namespace {

struct Fp4HostJob { const Tensor *tensor; const uint8_t *packed, *scales; const float *x_host; float *y_host; int rows, tokens; };

// Q/DQ of every job's activations, then the rows; `C` is shared.  Because the
// reference rejects a call whose activation is not finite, nothing is
// published unless the device status word stays zero.
int run_fp4_jobs(std::vector<Fp4HostJob> &jobs, int C) {
    Engine &e = g_engine;
    if (!g_state.fp8_is_ocp) { set_error("nvfp4: this device's fp8 converter is not OCP E4M3FN"); return -1; }
    if (salt_gpu_sync() != 0) return -1;
    size_t in_floats = 0, out_floats = 0;
    for (const Fp4HostJob &j : jobs) { in_floats += (size_t)j.tokens * C; out_floats += (size_t)j.tokens * j.rows; }
    const size_t bytes = (in_floats * 2 + out_floats) * 4 + 4096 + 512 * jobs.size();
    if (staging_reserve(bytes, bytes) != 0) return -1;
    int *st_dev = (int *)device_take(4);
    if (clear_words_launch(st_dev, 1, g_state.stream) != 0) return -1;
    std::vector<OutputCopy> copies;
    SaltGpuBatchStatsV2 &stats = e.stats;
    // Several single-token jobs: one activation pass per job, then all rows in ONE multi-matrix launch (streaming
    // rate instead of one latency-bound launch per matrix).  Otherwise job by job; a single token of a single job
    // runs its activation pass inside the rows' launch.
    bool all_single = jobs.size() > 1;
    for (const Fp4HostJob &j : jobs) all_single = all_single && j.tokens == 1;
    std::vector<SaltMi355Fp4Job> table;
    for (Fp4HostJob &j : jobs) {
        const size_t xin = (size_t)j.tokens * C, yout = (size_t)j.tokens * j.rows;
        float *x_dev = upload_activations(j.x_host, xin);
        if (!x_dev) return -1;
        float *dq_dev = (float *)device_take(xin * 4);
        uint8_t *y_dev = device_take(yout * 4), *y_pin = pinned_take(yout * 4);
        const bool one_launch = !all_single && j.tokens == 1 && C <= FP4_FUSED_MAX_COLS;
        if (g_state.tolerance_class && j.tokens <= 4) {
            // the tolerance-class kernel quantises the activation inside its launch
            if (salt_mi355_nvfp4_matvec_t_dev(j.packed, j.scales, j.tensor->stored_divisor, j.tensor->input_global_scale,
                                              j.rows, C, j.tokens, x_dev, (float *)y_dev, st_dev, g_state.stream) != 0)
                return -1;
        } else if (one_launch) {
            if (salt_mi355_nvfp4_matvec_qdq_dev(j.packed, j.scales, j.tensor->stored_divisor,
                                                j.tensor->input_global_scale, j.rows, C, x_dev, (float *)y_dev, st_dev, 0,
                                                g_state.stream) != 0)
                return -1;
        } else {
            if (salt_mi355_nvfp4_qdq_dev(x_dev, C, j.tokens, j.tensor->input_global_scale, nullptr, nullptr, dq_dev,
                                         st_dev, g_state.stream) != 0)
                return -1;
            if (all_single && !g_state.tolerance_class) {
                SaltMi355Fp4Job t;
                t.packed = j.packed; t.scales = j.scales; t.stored_divisor = j.tensor->stored_divisor;
                t.xs = dq_dev; t.ys = (float *)y_dev; t.rows = j.rows;
                table.push_back(t);
            } else if (salt_mi355_nvfp4_matvec_dev(j.packed, j.scales, j.tensor->stored_divisor, j.rows, C, j.tokens,
                                                   dq_dev, (float *)y_dev, 0, g_state.stream) != 0) {
                return -1;
            }
        }
        e.pending.push_back({y_pin, j.y_host, yout * 4});
        copies.push_back({y_dev, y_pin, yout * 4});
        stats.nvfp4_logical_packed_weight_bytes += (uint64_t)j.rows * C / 2;
        stats.nvfp4_logical_weight_scale_bytes += (uint64_t)j.rows * C / 16;
        stats.nvfp4_activation_input_bytes += xin * 4;
        stats.nvfp4_activation_qdq_bytes += xin * 4;
        stats.nvfp4_projection_output_bytes += yout * 4;
        stats.nvfp4_kernel_launches += one_launch ? 1 : all_single ? 1 : 2 + (uint64_t)((j.tokens - 1) / 4);
    }
    if (all_single && !table.empty()) {
        if (salt_mi355_nvfp4_jobs_dev(table.data(), (int)table.size(), C, 1, 0, g_state.stream) != 0) return -1;
        stats.nvfp4_kernel_launches += 1;
    }
    uint8_t *st_pin = pinned_take(4);
    for (const OutputCopy &c : copies)
        if (hip_ok(hipMemcpyAsync(c.pin, c.dev, c.nbytes, hipMemcpyDeviceToHost, g_state.stream), "output copy") != 0)
            return -1;
    if (hip_ok(hipMemcpyAsync(st_pin, st_dev, 4, hipMemcpyDeviceToHost, g_state.stream), "status copy") != 0 ||
        hip_ok(hipStreamSynchronize(g_state.stream), "nvfp4 sync") != 0)
        return -1;
    stats.nvfp4_completion_fences++;
    int status = 0;
    memcpy(&status, st_pin, 4);
    if (status != 0) {
        e.pending.clear();
        e.pinned_used = e.device_used = 0;
        set_error("nvfp4: an activation holds a non-finite value");
        return -1;
    }
    return salt_gpu_sync();
}

int fp4_job_for_key(const void *key, int R, int C, Fp4HostJob *job) {
    auto it = g_engine.tensors.find(key);
    if (!key || it == g_engine.tensors.end() || it->second.bits != 40 || it->second.R != R || it->second.C != C) {
        g_engine.stats.mapped_only_misses += g_engine.mapped_only ? 1 : 0;
        set_error("nvfp4: no NVFP4 tensor of %d x %d is registered under this key", R, C);
        return -1;
    }
    const Tensor &t = it->second;
    job->tensor = &t;
    job->packed = resident_address(t.vals, (size_t)R * C / 2);
    job->scales = resident_address(t.scales, (size_t)R * C / 16);
    if (!job->packed || !job->scales) { set_error("nvfp4: the tensor's resource is not active"); return -1; }
    job->rows = R;
    return 0;
}

}  // namespace

extern "C" {

int salt_gpu_nvfp4_matvec_batch(const void *key, int R, int C, int B, const float *inputs, float *outputs) {
    if (ready_or_fail("nvfp4_matvec_batch") != 0) return -1;
    if (!inputs || !outputs || R < 1 || C < 32 || C > MAX_C || B < 1 || (uint64_t)B * R > MAX_OUTPUT_FLOATS) {
        set_error("nvfp4_matvec_batch: bad arguments");
        return -1;
    }
    Fp4HostJob job = {};
    if (fp4_job_for_key(key, R, C, &job) != 0) return -1;
    job.x_host = inputs; job.y_host = outputs; job.tokens = B;
    std::vector<Fp4HostJob> jobs(1, job);
    if (run_fp4_jobs(jobs, C) != 0) { (void)salt_gpu_sync(); return -1; }
    return 0;
}

int salt_gpu_nvfp4_matvec(const void *key, int R, int C, const float *input, float *output) {
    return salt_gpu_nvfp4_matvec_batch(key, R, C, 1, input, output);
}

int salt_gpu_nvfp4_mixed_batch(const void *const *keys, const float *const *inputs, float *const *outputs,
                               const int *batches, const int *rows, int C, int njobs) {
    if (ready_or_fail("nvfp4_batch") != 0) return -1;
    if (!keys || !inputs || !outputs || !batches || !rows || njobs < 1 || (uint32_t)njobs > MAX_BATCH_JOBS || C < 32 ||
        C > MAX_C) {
        set_error("nvfp4_batch: bad arguments");
        return -1;
    }
    std::vector<Fp4HostJob> jobs;
    for (int j = 0; j < njobs; ++j) {
        Fp4HostJob job = {};
        if (!inputs[j] || !outputs[j] || batches[j] < 1 || rows[j] < 1 || fp4_job_for_key(keys[j], rows[j], C, &job) != 0)
            return -1;
        job.x_host = inputs[j]; job.y_host = outputs[j]; job.tokens = batches[j];
        jobs.push_back(job);
    }
    if (run_fp4_jobs(jobs, C) != 0) { (void)salt_gpu_sync(); return -1; }
    return 0;
}

int salt_gpu_nvfp4_batch(const void *const *keys, const float *const *inputs, float *const *outputs,
                         const int *batches, int R, int C, int njobs) {
    if (njobs < 1 || (uint32_t)njobs > MAX_BATCH_JOBS) return -1;
    std::vector<int> rows((size_t)njobs, R);
    return salt_gpu_nvfp4_mixed_batch(keys, inputs, outputs, batches, rows.data(), C, njobs);
}

// ================================================================ 8-bit affine (router gates) and bf16 (head)

int salt_gpu_q8_batch(const uint32_t *const *vals, const uint16_t *const *scales, const uint16_t *const *biases,
                      const float *const *xs, float *const *ys, const void *const *ids, const int *Rj, int C,
                      int njobs) {
    LegacyScope weights_of_this_call;
    if (ready_or_fail("q8_batch") != 0) return -1;
    if (!vals || !scales || !xs || !ys || !Rj || njobs < 1 || (uint32_t)njobs > MAX_BATCH_JOBS || C < 1 || C > MAX_C) {
        set_error("q8_batch: bad arguments");
        return -1;
    }
    std::vector<HostJob> jobs;
    int any_legacy = 0;
    size_t in_bytes = 0, out_bytes = 0;
    for (int j = 0; j < njobs; ++j) {
        const uint16_t *bias = biases ? biases[j] : nullptr;
        if (!vals[j] || !scales[j] || !xs[j] || !ys[j] || Rj[j] < 1) { set_error("q8_batch: job %d is malformed", j); return -1; }
        if (!key_agrees(ids ? ids[j] : nullptr, vals[j], scales[j], bias, Rj[j], C, 8)) {
            set_error("q8_batch: job %d does not match the tensor registered under its key", j);
            return -1;
        }
        // the engine sends one job per token of the same gate: contiguous rows of x and y become one job
        if (!jobs.empty()) {
            HostJob &prev = jobs.back();
            if (prev.rows == Rj[j] && vals[j] == vals[j - 1] && scales[j] == scales[j - 1] &&
                prev.x_host + (size_t)prev.tokens * C == xs[j] && prev.y_host + (size_t)prev.tokens * prev.rows == ys[j]) {
                prev.tokens++;
                continue;
            }
        }
        HostJob job = {};
        int legacy = 0;
        if (locate_q4(vals[j], scales[j], bias, Rj[j], C, &job.w, &legacy, 8) != 0) return -1;
        any_legacy |= legacy;
        job.x_host = xs[j]; job.y_host = ys[j]; job.rows = Rj[j]; job.tokens = 1;
        jobs.push_back(job);
    }
    for (const HostJob &j : jobs) {
        in_bytes += align_up((size_t)j.tokens * C * 4, 256);
        out_bytes += align_up((size_t)j.tokens * j.rows * 4, 256);
    }
    if (staging_reserve(in_bytes + out_bytes, in_bytes + out_bytes) != 0) return -1;
    std::vector<OutputCopy> copies;
    for (HostJob &j : jobs) {
        const float *x_dev = upload_activations(j.x_host, (size_t)j.tokens * C);
        if (!x_dev) { (void)salt_gpu_sync(); return -1; }
        const size_t count = (size_t)j.tokens * j.rows;
        uint8_t *dev = device_take(count * 4), *pin = pinned_take(count * 4);
        g_engine.pending.push_back({pin, j.y_host, count * 4});
        copies.push_back({dev, pin, count * 4});
        if (salt_mi355_q8_matvec_dev(j.w.vals, j.w.scales, j.w.biases, j.rows, C, j.tokens, x_dev, (float *)dev,
                                     g_state.stream) != 0) { (void)salt_gpu_sync(); return -1; }
    }
    count_batch(vals[0], any_legacy);
    return finish_call(copies);
}

int salt_gpu_q8_matvec(const uint32_t *vals, const uint16_t *scales, const uint16_t *biases, int R, int C,
                       const float *x, float *y) {
    LegacyScope weights_of_this_call;
    const void *id = vals;
    return salt_gpu_q8_batch(&vals, &scales, &biases, &x, &y, &id, &R, C, 1);
}

int salt_gpu_bf16_resource_slot(uint32_t kind, uint32_t resource_id, const void *key, const uint16_t *weights, int R,
                                int C) {
    if (ready_or_fail("bf16_resource_slot") != 0) return -1;
    if (R < 1 || C < 8 || (C & 7) != 0) { set_error("bf16_resource_slot: the column count must be a multiple of 8"); return -1; }
    Tensor t;
    t.bits = 16; t.R = R; t.C = C;
    return register_tensor(kind, resource_id, key, weights, (size_t)R * C * 2, nullptr, 0, nullptr, 0, t);
}

int salt_gpu_bf16_matvec(const void *key, int R, int C, const float *input, float *output) {
    if (ready_or_fail("bf16_matvec") != 0) return -1;
    auto it = g_engine.tensors.find(key);
    if (!key || it == g_engine.tensors.end() || it->second.bits != 16 || it->second.R != R || it->second.C != C ||
        R < 1 || C < 8 || (C & 7) != 0 || (size_t)R > MAX_OUTPUT_FLOATS || !input || !output) {
        g_engine.stats.mapped_only_misses += g_engine.mapped_only ? 1 : 0;
        set_error("bf16_matvec: no bf16 tensor of %d x %d is registered under this key, or bad arguments", R, C);
        return -1;
    }
    const Tensor &t = it->second;
    const uint8_t *weights = resident_address(t.vals, (size_t)R * C * 2);
    if (!weights) { set_error("bf16_matvec: the tensor's resource is not active"); return -1; }
    const size_t in_bytes = align_up((size_t)C * 4, 256), out_bytes = align_up((size_t)R * 4, 256);
    if (staging_reserve(in_bytes + out_bytes, in_bytes + out_bytes) != 0) return -1;
    const float *x_dev = upload_activations(input, (size_t)C);
    if (!x_dev) { (void)salt_gpu_sync(); return -1; }
    uint8_t *dev = device_take((size_t)R * 4), *pin = pinned_take((size_t)R * 4);
    g_engine.pending.push_back({pin, output, (size_t)R * 4});
    std::vector<OutputCopy> copies(1, OutputCopy{dev, pin, (size_t)R * 4});
    if (salt_mi355_bf16_matvec_dev(weights, R, C, 1, x_dev, nullptr, (float *)dev, g_state.stream) != 0) {
        (void)salt_gpu_sync();
        return -1;
    }
    const Resource &r = g_engine.resources[(size_t)t.resource];
    if (r.kind == KIND_EXPERT_LAYER) g_engine.stats.expert_layer_batches++; else g_engine.stats.trunk_batches++;
    g_engine.stats.direct_output_batches++;
    g_engine.stats.direct_output_jobs++;
    return finish_call(copies);
}

// ================================================================ whole-mapping conveniences of the reference ABI

// One mapped trunk range at a time (reference src/gpu_metal.m:1533-1536): trunk resource 0, copied to HBM.
int salt_gpu_resident_trunk_map(const void *base, size_t nbytes) {
    if (ready_or_fail("resident_trunk_map") != 0) return -1;
    const int ri = find_resource(1, 0);
    if (!base || nbytes < 1 || (ri >= 0 && g_engine.resources[(size_t)ri].active)) {
        set_error("resident_trunk_map: bad arguments, or a trunk range is already mapped");
        return -1;
    }
    return salt_gpu_weight_resource_bind(1, 0, base, nbytes);
}
int salt_gpu_resident_trunk_unmap(void) { return salt_gpu_weight_resource_unbind(1, 0); }   // reference gpu_hip.cpp:5180
// reference src/gpu_metal.m:1633-1642: the expert pool mapping is expert-layer resource 0
int salt_gpu_resident_pool_map(const void *base, size_t nbytes) { return salt_gpu_expert_resource_bind(0, base, nbytes); }

// ================================================================ fp32 cells over shared buffers

int salt_gpu_exact_cells(const SaltGpuExactCell *cells, int count) {
    if (ready_or_fail("exact_cells") != 0) return -1;
    if (!cells || count < 1 || count > 4096) { set_error("exact_cells: bad arguments"); return -1; }
    std::vector<SaltMi355Cell> table((size_t)count);
    for (int c = 0; c < count; ++c) {
        const SaltGpuExactCell &cell = cells[c];
        size_t elements[8] = {0};
        int views = 0;
        if (cell.n == 0) { set_error("exact_cells: cell %d is empty", c); return -1; }
        switch (cell.kind) {
        case SALT_GPU_EXACT_RMSNORM:
            if (cell.aux > 1u) { set_error("exact_cells: rmsnorm aux must be 0 or 1"); return -1; }
            views = 3; elements[0] = cell.n; elements[1] = cell.aux ? cell.n : 1u; elements[2] = cell.n;
            break;
        case SALT_GPU_EXACT_TOPK:
            if (cell.aux == 0 || cell.aux > cell.n) { set_error("exact_cells: topk aux must be in [1, n]"); return -1; }
            views = 4; elements[0] = elements[1] = cell.n; elements[2] = elements[3] = cell.aux;
            break;
        case SALT_GPU_EXACT_RESIDUAL_POSTNORM:
            views = 4; for (int k = 0; k < 4; ++k) elements[k] = cell.n;
            break;
        case SALT_GPU_EXACT_PARALLEL_COMBINE:
            views = 8; for (int k = 0; k < 8; ++k) elements[k] = k == 6 ? (size_t)cell.n * 2u : cell.n;
            break;
        case SALT_GPU_EXACT_SOFTCAP:
            if (!(cell.scalar > 0.0f) || !isfinite(cell.scalar)) { set_error("exact_cells: softcap needs a positive cap"); return -1; }
            views = 1; elements[0] = cell.n;
            break;
        case SALT_GPU_EXACT_ROUTER_INPUT:
            views = 3; for (int k = 0; k < 3; ++k) elements[k] = cell.n;
            break;
        default:
            set_error("exact_cells: cell %d has unknown kind %d", c, (int)cell.kind);
            return -1;
        }
        SaltMi355Cell &out = table[(size_t)c];
        memset(&out, 0, sizeof out);
        out.kind = (int)cell.kind; out.n = cell.n; out.aux = cell.aux; out.eps = cell.eps; out.scalar = cell.scalar;
        for (int k = 0; k < views; ++k) {
            const SaltGpuSharedBuffer *b = cell.views[k];
            // element offsets and capacities count floats (ints for the selection of TOPK have the same size)
            const size_t capacity = b && b->contents ? b->nbytes / sizeof(float) : 0;
            if (!b || !b->contents || cell.offsets[k] > capacity || elements[k] > capacity - cell.offsets[k]) {
                set_error("exact_cells: cell %d view %d lies outside its buffer", c, k);
                return -1;
            }
            uint8_t *dev = (uint8_t *)shared_device_view(b->contents, b->nbytes);
            if (!dev) { set_error("exact_cells: cell %d view %d is not a shared buffer of this backend", c, k); return -1; }
            out.views[k] = dev + cell.offsets[k] * sizeof(float);
        }
    }
    if (staging_reserve(256, 256) != 0) return -1;
    int *status_dev = (int *)device_take(256), *status_pin = (int *)pinned_take(256);
    *status_pin = -1;
    if (clear_words_launch(status_dev, 2, g_state.stream) != 0 ||
        salt_mi355_cells_dev(table.data(), count, status_dev, g_state.stream) != 0 ||
        hip_ok(hipMemcpyAsync(status_pin, status_dev, sizeof(int), hipMemcpyDeviceToHost, g_state.stream),
               "exact_cells status") != 0) {
        (void)salt_gpu_sync();
        return -1;
    }
    if (salt_gpu_sync() != 0) return -1;          // one status-bearing completion for the whole sequence
    if (*status_pin != 0) { set_error("exact_cells: a cell met a non-finite input or result"); return -1; }
    return 0;
}

// ================================================================ residency operations

// Gives back everything create took.  Used by destroy and by every failure inside create, so that a half-built
// arena never lingers.
static int residency_release(Residency &r) {
    int failed = 0;
    for (Residency::StagingBuffer &b : r.buffers)
        if (b.copied) failed |= hip_ok(hipEventDestroy(b.copied), "residency: destroy event");
    for (hipStream_t &lane : r.lanes)
        if (lane) failed |= hip_ok(hipStreamDestroy(lane), "residency: destroy copy stream");
    if (r.pinned) failed |= hip_ok(hipHostFree(r.pinned), "residency: free staging");
    if (r.arena) failed |= hip_ok(hipFree(r.arena), "residency: free arena");
    r = Residency();
    return failed;
}

static int res_create(void *, const SaltGpuResidencyPlan *plan) {
    Residency &r = g_engine.residency;
    if (!g_state.ready) { set_error("residency: the backend is not initialised"); return -1; }
    if (r.live || r.broken) { set_error("residency: an arena exists already (destroy it first)"); return -1; }
    if (!plan) { set_error("residency: no plan"); return -1; }
    const uint64_t seats_bytes = (uint64_t)plan->slot_count * plan->slot_bytes;
    const bool shaped = plan->slot_count >= 1 && plan->staging_count >= 1 && plan->slot_bytes >= 1 &&
                        plan->staging_bytes >= plan->slot_bytes && plan->device_budget_bytes >= 1;
    const bool fits = shaped && plan->slot_base_offset <= plan->device_budget_bytes &&
                      seats_bytes <= plan->device_budget_bytes - plan->slot_base_offset;
    if (!fits) { set_error("residency: the plan's seats do not fit its device budget"); return -1; }
    r = Residency();
    r.plan = *plan;
    int ok = hip_ok(hipMalloc((void **)&r.arena, plan->device_budget_bytes), "residency: arena in HBM") == 0 &&
             hip_ok(hipHostMalloc((void **)&r.pinned, (size_t)plan->staging_bytes * plan->staging_count, hipHostMallocDefault),
                    "residency: pinned staging") == 0;
    for (int l = 0; ok && l < Residency::kLanes; ++l)
        ok = hip_ok(hipStreamCreateWithFlags(&r.lanes[l], hipStreamNonBlocking), "residency: copy stream") == 0;
    if (ok) r.buffers.assign(plan->staging_count, Residency::StagingBuffer());
    for (size_t b = 0; ok && b < r.buffers.size(); ++b)
        ok = hip_ok(hipEventCreateWithFlags(&r.buffers[b].copied, hipEventDisableTiming), "residency: copy event") == 0;
    if (!ok) {
        char keep[sizeof g_state.last_error];
        memcpy(keep, g_state.last_error, sizeof keep);
        (void)residency_release(r);
        memcpy(g_state.last_error, keep, sizeof keep);
        return -1;
    }
    r.seat_buffer.assign(plan->slot_count, Residency::kNone);
    r.live = 1;
    return 0;
}

static int res_staging(void *, uint32_t staging_slot, void **address, size_t *capacity) {
    Residency &r = g_engine.residency;
    if (!r.live || r.broken || !address || !capacity || staging_slot >= r.buffers.size()) return -1;
    *address = r.staging_at(staging_slot);
    *capacity = (size_t)r.plan.staging_bytes;
    return 0;
}

// The staging buffer holds the seat's bytes (the engine's read callback filled it): start the copy into the seat.
static int res_populate(void *, uint32_t slot, uint64_t device_offset, uint32_t staging_slot, size_t nbytes,
                        uint64_t ticket) {
    Residency &r = g_engine.residency;
    if (!r.live || r.broken || ticket == 0 || nbytes == 0 || nbytes > r.plan.slot_bytes) return -1;
    if (slot >= r.seat_buffer.size() || staging_slot >= r.buffers.size()) return -1;
    if (device_offset != r.plan.slot_base_offset + (uint64_t)slot * r.plan.slot_bytes) return -1;   // a seat's own place
    Residency::StagingBuffer &buffer = r.buffers[staging_slot];
    if (buffer.ticket != 0 || r.seat_buffer[slot] != Residency::kNone) return -1;    // either side is still busy
    const hipStream_t lane = r.lane_of(staging_slot);
    if (hip_ok(hipMemcpyAsync(r.arena + device_offset, r.staging_at(staging_slot), nbytes, hipMemcpyHostToDevice, lane),
               "residency: seat copy") != 0)
        return -1;
    if (hip_ok(hipEventRecord(buffer.copied, lane), "residency: seat copy event") != 0) {
        // the copy is queued but cannot be observed: wait it out so that the buffer may be reused, or give up
        if (hipStreamSynchronize(lane) != hipSuccess) r.broken = 1;
        return -1;
    }
    buffer.ticket = ticket;
    buffer.seat = slot;
    r.seat_buffer[slot] = staging_slot;
    return 0;
}

static int res_poll(void *, uint32_t slot, uint64_t ticket, int *complete) {
    Residency &r = g_engine.residency;
    if (!r.live || r.broken || !complete || ticket == 0 || slot >= r.seat_buffer.size()) return -1;
    const uint32_t b = r.seat_buffer[slot];
    if (b == Residency::kNone || r.buffers[b].ticket != ticket || r.buffers[b].seat != slot) return -1;
    const hipError_t state = hipEventQuery(r.buffers[b].copied);
    if (state == hipErrorNotReady) { *complete = 0; return 0; }
    if (state != hipSuccess) return hip_ok(state, "residency: seat copy");
    r.buffers[b].ticket = 0;
    r.buffers[b].seat = Residency::kNone;
    r.seat_buffer[slot] = Residency::kNone;
    *complete = 1;
    return 0;
}

static int res_resolve(void *, uint64_t device_offset, size_t nbytes, uintptr_t *address) {
    Residency &r = g_engine.residency;
    if (!r.live || r.broken || !address || nbytes == 0) return -1;
    if (device_offset > r.plan.device_budget_bytes || nbytes > r.plan.device_budget_bytes - device_offset) return -1;
    *address = (uintptr_t)(r.arena + device_offset);
    return 0;
}

// The seat is about to be given to another expert: a fill that is still running must end, and no kernel may still
// read the old bytes.
static int res_retire(void *, uint32_t slot, uint64_t) {
    Residency &r = g_engine.residency;
    if (!r.live || r.broken || slot >= r.seat_buffer.size()) return -1;
    const uint32_t b = r.seat_buffer[slot];
    if (b != Residency::kNone) {
        if (b >= r.buffers.size() || r.buffers[b].seat != slot) return -1;
        if (hip_ok(hipEventSynchronize(r.buffers[b].copied), "residency: retire waits for the fill") != 0) return -1;
        r.buffers[b].ticket = 0;
        r.buffers[b].seat = Residency::kNone;
        r.seat_buffer[slot] = Residency::kNone;
    }
    if (salt_gpu_sync() != 0 || drain_device() != 0) return -1;
    return 0;
}

static int res_destroy(void *) {
    Residency &r = g_engine.residency;
    if (!r.live && !r.broken) return -1;
    int failed = drain_device();
    for (Seat &s : g_engine.seats)
        if (s.active && s.resident) { g_engine.logical_seat[(size_t)s.logical_id] = -1; s = Seat(); }
    if (r.published) {                                       // the spans leave with the arena (reference gpu_hip.cpp:750-769)
        for (Region &g : g_engine.regions) { g.device = nullptr; g.arena_offset = 0; g.populated = 0; }
        g_engine.pool_bytes = 0;
        g_engine.pool_final = 0;
    }
    g_engine.pool_layout_bytes = g_engine.pool_layout_max_span = 0;
    g_engine.pool_span_count = 0;
    failed |= residency_release(r);
    return failed ? -1 : 0;
}

// Permanent spans: the regions of the component pool, laid out at the front of the arena (reference
// gpu_hip.cpp:3429-3571).  The engine reads each span through the callback below into a staging slot and has it
// copied chunk by chunk; publish makes the tensors inside resolvable.
static int pool_source_read(void *context, uint64_t source_offset, void *destination, size_t nbytes) {
    const size_t index = (size_t)(uintptr_t)context - 1;          // the span index travels in the pointer
    if (!context || index >= g_engine.regions.size() || !destination || nbytes == 0) return -1;
    const Region &g = g_engine.regions[index];
    if (!g.host || source_offset < g.source_offset) return -1;
    const uint64_t local = source_offset - g.source_offset;
    if (local > g.nbytes || nbytes > g.nbytes - local) return -1;
    memcpy(destination, g.host + local, nbytes);
    return 0;
}

static int res_permanent_layout(void *, SaltGpuResidencyPermanentLayout *layout, size_t layout_size) {
    Engine &e = g_engine;
    if (!g_state.ready || !layout || layout_size != sizeof *layout || e.pool_final) return -1;
    if (e.pool_span_count == 0) {
        if (pool_build_regions() != 0) {
            set_error("permanent layout: no tensor is registered in a pool-bound resource");
            return -1;
        }
        uint64_t cursor = 0, maximum = 0;
        for (Region &g : e.regions) {
            cursor = (cursor + POOL_ALIGN - 1) / POOL_ALIGN * POOL_ALIGN;
            g.arena_offset = cursor;
            g.populated = 0;
            g.device = nullptr;
            cursor += g.nbytes;
            if (g.nbytes > maximum) maximum = g.nbytes;
        }
        e.pool_layout_bytes = cursor;
        e.pool_layout_max_span = maximum;
        e.pool_span_count = (uint32_t)e.regions.size();
    }
    layout->permanent_bytes = e.pool_layout_bytes;
    layout->maximum_span_bytes = e.pool_layout_max_span;
    layout->span_count = e.pool_span_count;
    layout->alignment = (uint32_t)POOL_ALIGN;
    return 0;
}

static int res_permanent_span(void *, uint32_t span_index, SaltGpuResidencyPermanentSpan *span, size_t span_size) {
    Engine &e = g_engine;
    if (!span || span_size != sizeof *span || span_index >= e.pool_span_count || span_index >= e.regions.size()) return -1;
    const Region &g = e.regions[span_index];
    if (g.resource < 0 || (size_t)g.resource >= e.resources.size()) return -1;
    const Resource &r = e.resources[(size_t)g.resource];
    if (!r.active || !r.pool) return -1;
    memset(span, 0, sizeof *span);
    span->source.resource.kind = r.kind;
    span->source.resource.resource_id = r.id;
    span->source.source_offset = g.source_offset;
    span->source.nbytes = g.nbytes;
    span->source.read = pool_source_read;
    span->source.read_context = (void *)(uintptr_t)(span_index + 1u);
    span->device_offset = g.arena_offset;
    return 0;
}

static int res_permanent_copy(void *, uint32_t span_index, uint64_t device_offset, uint32_t staging_slot, size_t nbytes,
                              uint64_t ticket) {
    Engine &e = g_engine;
    Residency &r = e.residency;
    if (!r.live || r.broken || r.published || ticket == 0 || nbytes == 0 || span_index >= e.pool_span_count ||
        span_index >= e.regions.size() || staging_slot >= r.plan.staging_count || nbytes > r.plan.staging_bytes)
        return -1;
    Region &g = e.regions[span_index];
    if (device_offset != g.arena_offset + g.populated || nbytes > g.nbytes - g.populated ||
        device_offset > r.plan.permanent_bytes || nbytes > r.plan.permanent_bytes - device_offset) {
        set_error("permanent copy: chunks of a span arrive in order and stay inside the permanent part of the arena");
        return -1;
    }
    const hipStream_t lane = r.lane_of(staging_slot);
    if (r.buffers[staging_slot].ticket != 0) return -1;      // a seat fill still reads this buffer
    if (hip_ok(hipMemcpyAsync(r.arena + device_offset, r.staging_at(staging_slot), nbytes, hipMemcpyHostToDevice, lane),
               "permanent span copy") != 0)
        return -1;
    if (hip_ok(hipStreamSynchronize(lane), "permanent span copy") != 0) { r.broken = 1; return -1; }
    g.populated += nbytes;                                   // the staging slot is free again on return
    return 0;
}

static int res_permanent_publish(void *) {
    Engine &e = g_engine;
    Residency &r = e.residency;
    if (!r.live || r.broken || r.published || e.pool_span_count == 0 || e.pool_span_count != e.regions.size()) return -1;
    uint64_t total = 0;
    for (const Region &g : e.regions)
        if (g.populated != g.nbytes || g.arena_offset > r.plan.permanent_bytes ||
            g.nbytes > r.plan.permanent_bytes - g.arena_offset) {
            set_error("permanent publish: a span is not fully populated");
            return -1;
        }
    for (Region &g : e.regions) { g.device = r.arena + g.arena_offset; total += g.nbytes; }
    e.pool_bytes = total;
    if (total > e.pool_peak_bytes) e.pool_peak_bytes = total;
    e.pool_final = 1;
    r.published = 1;
    return 0;
}

static const SaltGpuResidencyBackendOps residency_ops = {
    SALT_GPU_RESIDENCY_ABI_VERSION, sizeof(SaltGpuResidencyBackendOps),
    res_create, res_staging, res_populate, res_poll, res_resolve, res_retire, res_destroy,
    res_permanent_layout, res_permanent_span, res_permanent_copy, res_permanent_publish,
};

const SaltGpuResidencyBackendOps *salt_gpu_residency_backend_ops(void) { return &residency_ops; }

// ================================================================ off-path entry points (null-backend answers)

// The ROCm backend of the reference leaves the batched bf16 matvec to the CPU (src/gpu_hip.cpp:4624-4628); its CUDA
// counterpart computes a different, single-chain order for the vision tower.
int salt_gpu_bf16_matvec_batch(const void *, int, int, int, const float *, float *) { return -1; }
const struct SaltGpuDispatch *salt_dispatch_get(void) { return nullptr; }
const struct SaltTextGpuProgramOps *salt_gpu_tensor_program_ops(void) { return nullptr; }
int salt_gpu_attention_batch(int, int, int, int, int, const SaltGpuSharedBuffer *, size_t, const SaltGpuSharedBuffer *,
                             size_t, size_t, int, int, int, int, SaltGpuSharedBuffer *, size_t, SaltGpuSharedBuffer *,
                             size_t, size_t, int) { return -1; }
int salt_gpu_attention_prepare(const SaltGpuSharedBuffer *) { return -1; }
int salt_gpu_attention_bind_kv(size_t, size_t, int) { return -1; }
int salt_gpu_attention_materialize(SaltGpuSharedBuffer *, int, uint64_t *copied) { if (copied) *copied = 0; return -1; }
int salt_gpu_attention_import(SaltGpuSharedBuffer *, int, uint64_t *copied) { if (copied) *copied = 0; return -1; }
int salt_gpu_attention_rewind(int) { return -1; }
int salt_gpu_attention_transform(int, int, int, int, int, int, int, int, float, SaltGpuSharedBuffer *, size_t,
                                 SaltGpuSharedBuffer *, size_t, SaltGpuSharedBuffer *, size_t, const float *,
                                 const float *, const float *, const float *, int, SaltGpuSharedBuffer *, size_t,
                                 size_t) { return -1; }

}  // extern "C"
