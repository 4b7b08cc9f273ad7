/* Expert residency through the engine's own path, against this repository's backend.
 *
 * The engine side is the reference's, compiled from its sources where they lie: the packed expert pool
 * (src/st.c:154), the expert cache with its resource hooks (src/cache.c:968, 1338-1358), the residency ledger
 * (src/gpu_residency.c) and the CPU kernels that give the expected values (src/kernels.c).  This program plays the
 * model's part the way models/gemma4-26b-a4b/src/gemma4_text.c does (init_full_gpu :2644-2790,
 * g4_init_device_residency :2576-2642, g4_selected_cache_bind_resident :1886-1980, the unbind hook :1982-2000):
 *
 *   trunk mapping  -> describe, activate as a bounded window, pool-bind, register the tensors
 *   residency      -> permanent layout, plan (one seat per (layer, expert) of the pool), init, populate the
 *                     permanent spans through staging, publish
 *   expert cache   -> zero-copy cache over the pool file; its bind hook populates a seat (begin, poll, acquire,
 *                     resolve), publishes it with salt_gpu_selected_resource_bind_resident and releases the lease;
 *                     its unbind hook unbinds and retires
 *   decode         -> trunk projections and the selected expert chain run on the device from those addresses only
 *                     (mapped-only mode) and are compared bit for bit with the CPU kernels
 *
 * Phase 1 seats every expert of every layer (30 x 128 by default: the whole pool lives in HBM).  Phase 2 reopens the
 * ledger with 16 seats so that the cache has to evict, and checks the chain again after the seats have turned over.
 *
 * usage: residency-engine-path [layers [directory-for-the-pool-file]]
 * Only two layers of the pool file carry data; the others are holes in a sparse file (all-zero weights), which
 * costs the same traffic to seat.
 */
#include "salt/gpu.h"
#include "salt/gpu_residency.h"
#include "salt/kernels.h"
#include "salt/salt.h"
#include "gemma4.h"

/* device-to-host copy helper of the backend library (include/salt_gpu_mi355.h) */
int salt_mi355_dev_download(void *host_dst, const void *device_src, size_t nbytes);

#include <fcntl.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <sys/stat.h>
#include <time.h>
#include <unistd.h>

enum { HIDDEN = 2816, ROUTED = 704, DENSE = 2112, EXPERTS = 128, TOPK = 8, HEADER = 24 };
#define PROJ_VALS   ((size_t)ROUTED * HIDDEN / 2)
#define PROJ_META   ((size_t)ROUTED * HIDDEN / 64 * 2)
#define PROJ_BYTES  (PROJ_VALS + 2 * PROJ_META)
#define SLOT_BYTES  (3 * PROJ_BYTES)                 /* 3,345,408 */

#define CHECK(x) do { if (!(x)) { fprintf(stderr, "residency-engine-path: check failed at line %d: %s\n", \
                                          __LINE__, #x); return 1; } } while (0)

static double now_s(void) {
    struct timespec t;
    clock_gettime(CLOCK_MONOTONIC, &t);
    return (double)t.tv_sec + 1e-9 * (double)t.tv_nsec;
}

static uint64_t rng_state;
static uint32_t rng(void) {
    rng_state = rng_state * 6364136223846793005ull + 1442695040888963407ull;
    return (uint32_t)(rng_state >> 32);
}
static uint16_t bf16_of(float f) { uint32_t u; memcpy(&u, &f, 4); return (uint16_t)((u + 0x7fffu + ((u >> 16) & 1u)) >> 16); }

/* values, then scales, then biases of one affine tensor with `elements` weights */
static void fill_affine(uint8_t *p, size_t elements, int bits) {
    const size_t vb = bits == 4 ? elements / 2 : elements, groups = elements / 64;
    uint16_t *scales = (uint16_t *)(p + vb), *biases = scales + groups;
    for (size_t i = 0; i < vb / 4; i++) ((uint32_t *)p)[i] = rng();
    for (size_t g = 0; g < groups; g++) {
        const float s = (0.002f + 0.02f * (float)(rng() & 1023) / 1024.0f) * ((rng() & 8) ? 1.0f : -1.0f);
        scales[g] = bf16_of(bits == 4 ? s : s / 16.0f);
        biases[g] = bf16_of(-s * (bits == 4 ? 7.5f : 8.0f) + 0.001f * (float)((int)(rng() & 15) - 8));
    }
}

static void fill_x(float *x, int n) { for (int i = 0; i < n; i++) x[i] = ((float)(rng() & 0xffff) / 32768.0f - 1.0f) * 1.5f; }

/* ---- the model's side of the hooks --------------------------------------------------------------------------- */

typedef struct Model {
    SaltGpuResidency residency;
    void *arena;
    uint64_t generation;
    uint64_t binds, unbinds, fences;
} Model;

static int payload_read(void *context, uint64_t source_offset, void *destination, size_t nbytes) {
    if (!context || !destination || nbytes == 0 || source_offset != 0) return -1;
    memcpy(destination, context, nbytes);
    return 0;
}

static int hook_bind(void *opaque, int slot, int layer, int expert, const void *base, size_t nbytes, const void *payload) {
    Model *m = (Model *)opaque;
    SaltGpuResidencySource source;
    SaltGpuResidencyBinding binding;
    uintptr_t device_address = 0;
    uint64_t ticket = 0;
    const uint64_t logical = (uint64_t)layer * EXPERTS + (uint64_t)expert;
    int polled;
    if (!m || !base || !payload || nbytes < SLOT_BYTES || slot < 0) return -1;
    const uint64_t generation = ++m->generation;
    const uint32_t staging_slot = (uint32_t)((generation - 1u) % m->residency.plan.staging_count);
    memset(&source, 0, sizeof source);
    source.resource.kind = SALT_GPU_RESOURCE_EXPERT_LAYER;
    source.resource.resource_id = (uint32_t)logical;
    source.logical_resource_id = logical;
    source.nbytes = SLOT_BYTES;
    source.read = payload_read;
    source.read_context = (void *)payload;
    if (salt_gpu_residency_population_begin(&m->residency, (uint32_t)slot, generation, &source, staging_slot, &ticket) != 0)
        return -1;
    do polled = salt_gpu_residency_population_poll(&m->residency, (uint32_t)slot, logical, generation, ticket);
    while (polled == 0);
    if (polled != 1 || salt_gpu_residency_acquire(&m->residency, (uint32_t)slot, logical, generation, &binding) != 1)
        return -1;
    if (salt_gpu_residency_resolve(&m->residency, &binding, &device_address) != 0 ||
        salt_gpu_selected_resource_bind_resident(slot, logical, payload, SLOT_BYTES, device_address, generation) != 0) {
        (void)salt_gpu_residency_release(&m->residency, &binding);
        return -1;
    }
    m->binds++;
    return salt_gpu_residency_release(&m->residency, &binding);
}

static int hook_fence(void *opaque) {
    ((Model *)opaque)->fences++;
    return salt_gpu_selected_resources_fence();
}

static int hook_unbind(void *opaque, int slot, int layer, int expert) {
    Model *m = (Model *)opaque;
    const uint64_t logical = (uint64_t)layer * EXPERTS + (uint64_t)expert;
    SaltGpuResidencySlot *seat;
    if (!m || slot < 0 || (uint32_t)slot >= m->residency.plan.slot_count) return -1;
    seat = &m->residency.slots[slot];
    if (seat->state != SALT_GPU_RESIDENCY_READY || seat->logical_resource_id != logical || seat->lease_count != 0 ||
        salt_gpu_selected_resource_unbind(slot, logical) != 0)
        return -1;
    m->unbinds++;
    return salt_gpu_residency_retire(&m->residency, (uint32_t)slot, logical, seat->generation);
}

static int open_residency(Model *m, uint32_t seats, uint32_t staging_count, int with_permanent,
                          SaltGpuResidencyPermanentLayout *layout) {
    const SaltGpuResidencyBackendOps *ops = salt_gpu_residency_backend_ops();
    SaltGpuResidencyPlan plan;
    size_t arena_bytes;
    uint64_t slot_base = 0;
    if (!ops) return -1;
    memset(layout, 0, sizeof *layout);
    if (with_permanent) {
        if (salt_gpu_residency_permanent_layout(ops, NULL, layout, sizeof *layout) != 0) return -1;
        slot_base = (layout->permanent_bytes + layout->alignment - 1u) / layout->alignment * layout->alignment;
    }
    memset(&plan, 0, sizeof plan);
    plan.device_budget_bytes = slot_base + (uint64_t)seats * SLOT_BYTES;
    plan.permanent_bytes = layout->permanent_bytes;
    plan.slot_base_offset = slot_base;
    plan.slot_bytes = SLOT_BYTES;
    plan.staging_bytes = SLOT_BYTES;
    plan.slot_count = seats;
    plan.staging_count = staging_count;
    plan.device_alignment = with_permanent ? layout->alignment : 256u;
    arena_bytes = salt_gpu_residency_arena_requirement(&plan);
    if (arena_bytes == 0 || !(m->arena = calloc(1u, arena_bytes))) return -1;
    if (salt_gpu_residency_init(&m->residency, &plan, ops, NULL, m->arena, arena_bytes) != 0) return -1;
    if (with_permanent && salt_gpu_residency_populate_permanent(&m->residency) != 0) return -1;
    return 0;
}

/* ---- expected values on the CPU and the device chain --------------------------------------------------------- */

static void cpu_expert(const uint8_t *payload, const float *x, float *out) {
    static float gate[ROUTED], up[ROUTED];
    const uint8_t *p[3] = {payload, payload + PROJ_BYTES, payload + 2 * PROJ_BYTES};
    salt_q4_matvec((const uint32_t *)p[0], (const uint16_t *)(p[0] + PROJ_VALS), (const uint16_t *)(p[0] + PROJ_VALS + PROJ_META),
                   ROUTED, HIDDEN, x, gate);
    salt_q4_matvec((const uint32_t *)p[1], (const uint16_t *)(p[1] + PROJ_VALS), (const uint16_t *)(p[1] + PROJ_VALS + PROJ_META),
                   ROUTED, HIDDEN, x, up);
    for (int i = 0; i < ROUTED; i++) gate[i] = salt_gemma4_gelu_tanh(gate[i]) * up[i];
    salt_q4_matvec((const uint32_t *)p[2], (const uint16_t *)(p[2] + PROJ_VALS), (const uint16_t *)(p[2] + PROJ_VALS + PROJ_META),
                   HIDDEN, ROUTED, gate, out);
}

typedef struct Buffers { SaltGpuSharedBuffer in, out, gate, up; } Buffers;

/* the selected chain of one token over `count` experts of `layer` (ascending), all from their seats */
static int device_chain(SaltCache *cache, Buffers *b, int layer, const int *experts, int count, const float *x,
                        const char *what) {
    int slots[TOPK];
    const uint8_t *payloads[TOPK];
    SaltGpuMoeExpert records[TOPK];
    static float want[HIDDEN];
    if (salt_cache_getmany(cache, layer, experts, count, slots) < 0) return -1;
    if (salt_cache_acquire_many(cache, slots, layer, experts, count, payloads) != 0) return -1;
    memset(records, 0, sizeof records);
    for (int i = 0; i < count; i++) {
        const uint8_t *p[3] = {payloads[i], payloads[i] + PROJ_BYTES, payloads[i] + 2 * PROJ_BYTES};
        const uint32_t **vals[3] = {&records[i].gate_vals, &records[i].up_vals, &records[i].down_vals};
        const uint16_t **scales[3] = {&records[i].gate_scales, &records[i].up_scales, &records[i].down_scales};
        const uint16_t **biases[3] = {&records[i].gate_biases, &records[i].up_biases, &records[i].down_biases};
        const void **ids[3] = {&records[i].gate_id, &records[i].up_id, &records[i].down_id};
        for (int k = 0; k < 3; k++) {
            *vals[k] = (const uint32_t *)p[k];
            *scales[k] = (const uint16_t *)(p[k] + PROJ_VALS);
            *biases[k] = (const uint16_t *)(p[k] + PROJ_VALS + PROJ_META);
            *ids[k] = p[k];
        }
        records[i].group = 1;
        records[i].resource_slot = slots[i];
        records[i].logical_resource_id = (uint64_t)layer * EXPERTS + (uint64_t)experts[i];
        memcpy((float *)b->in.contents + (size_t)i * HIDDEN, x, sizeof(float) * HIDDEN);
    }
    if (salt_gpu_q4_moe_chain_selected(records, count, HIDDEN, ROUTED, (const float *)b->in.contents,
            (float *)b->out.contents, (float *)b->gate.contents, (float *)b->up.contents, (size_t)count * ROUTED) != 0 ||
        salt_gpu_sync() != 0) {
        fprintf(stderr, "residency-engine-path: %s: the device chain failed\n", what);
        return -1;
    }
    for (int i = 0; i < count; i++) {
        cpu_expert(payloads[i], x, want);
        if (memcmp(want, (const float *)b->out.contents + (size_t)i * HIDDEN, sizeof want) != 0) {
            fprintf(stderr, "residency-engine-path: %s: layer %d expert %d differs from the CPU kernels\n", what, layer,
                    experts[i]);
            return -1;
        }
    }
    return salt_cache_release_many(cache, slots, layer, experts, count);
}

/* ---- trunk mapping -------------------------------------------------------------------------------------------- */

typedef struct TrunkTensor { size_t offset; int rows, cols, bits; } TrunkTensor;

int main(int argc, char **argv) {
    const int layers = argc > 1 ? atoi(argv[1]) : 30;
    const char *directory = argc > 2 ? argv[2] : "/tmp";
    char path[512];
    Model model;
    SaltCfg cfg;
    SaltExpertPool pool;
    SaltCache cache;
    SaltGpuResidencyPermanentLayout layout;
    SaltGpuResidencyStats stats;
    SaltGpuWeightResourceUsage usage;
    Buffers b;
    static float x[HIDDEN], got[HIDDEN], want[HIDDEN];
    double t0, t1;

    if (getenv("SALT_REQUIRE_GPU") == NULL && salt_gpu_init() != 0) { puts("residency-engine-path: SKIP (no device)"); return 0; }
    CHECK(layers >= 2 && layers <= 64);
    CHECK(salt_gpu_init() == 0);
    CHECK(SLOT_BYTES == 3345408u);
    rng_state = 0x5a17c0de;
    memset(&model, 0, sizeof model);
    const int real_layers[2] = {0, layers - 1 - (layers > 2)};

    /* the pool file: header, then layers x experts seats; two layers carry data */
    snprintf(path, sizeof path, "%s/salt-residency-pool-%ld.bin", directory, (long)getpid());
    {
        const uint64_t header[3] = {SLOT_BYTES, (uint64_t)layers, EXPERTS};
        uint8_t *seat = malloc(SLOT_BYTES);
        int fd = open(path, O_CREAT | O_TRUNC | O_RDWR, 0600);
        CHECK(fd >= 0 && seat);
        CHECK(ftruncate(fd, (off_t)(HEADER + (uint64_t)layers * EXPERTS * SLOT_BYTES)) == 0);
        CHECK(pwrite(fd, header, sizeof header, 0) == (ssize_t)sizeof header);
        for (int r = 0; r < 2; r++)
            for (int e = 0; e < EXPERTS; e++) {
                for (int k = 0; k < 3; k++) fill_affine(seat + (size_t)k * PROJ_BYTES, (size_t)ROUTED * HIDDEN, 4);
                CHECK(pwrite(fd, seat, SLOT_BYTES, (off_t)(HEADER + ((uint64_t)real_layers[r] * EXPERTS + (uint64_t)e) * SLOT_BYTES))
                      == (ssize_t)SLOT_BYTES);
            }
        free(seat);
        CHECK(close(fd) == 0);
    }
    memset(&cfg, 0, sizeof cfg);
    cfg.n_layers = layers; cfg.n_experts = EXPERTS; cfg.expert_nbytes = SLOT_BYTES;
    CHECK(salt_pool_open_packed(&pool, path, &cfg) == 0);
    CHECK(unlink(path) == 0);                           /* the mapping keeps the file until the pool closes */

    /* the trunk mapping: two layers of dense gate / up / down (Q4) and a router gate (8-bit), with unrelated bytes
     * between the layers, so the pool holds more than one region */
    TrunkTensor trunk[8];
    size_t trunk_bytes = 0;
    for (int l = 0; l < 2; l++) {
        const int rows[4] = {DENSE, DENSE, HIDDEN, EXPERTS}, cols[4] = {HIDDEN, HIDDEN, DENSE, HIDDEN}, bits[4] = {4, 4, 4, 8};
        trunk_bytes += 40;                              /* tensors sit at odd multiples of eight, like the pool file */
        for (int k = 0; k < 4; k++) {
            const size_t elements = (size_t)rows[k] * cols[k];
            trunk[l * 4 + k] = (TrunkTensor){trunk_bytes, rows[k], cols[k], bits[k]};
            trunk_bytes += (bits[k] == 4 ? elements / 2 : elements) + elements / 64 * 4;
        }
        trunk_bytes += 3u << 20;                        /* norms, attention: nothing this backend is given */
    }
    uint8_t *trunk_map = NULL;
    CHECK(posix_memalign((void **)&trunk_map, 4096, trunk_bytes) == 0);
    memset(trunk_map, 0xA5, trunk_bytes);
    for (int i = 0; i < 8; i++) fill_affine(trunk_map + trunk[i].offset, (size_t)trunk[i].rows * trunk[i].cols, trunk[i].bits);

    /* init_full_gpu */
    salt_gpu_set_mapped_only(1);
    CHECK(salt_gpu_weight_resource_describe(SALT_GPU_RESOURCE_TRUNK, 0, trunk_map, trunk_bytes) == 0);
    CHECK(salt_gpu_weight_resource_pool_bind(SALT_GPU_RESOURCE_TRUNK, 0) != 0);            /* not active yet */
    CHECK(salt_gpu_weight_resource_activate(SALT_GPU_RESOURCE_TRUNK, 0, SALT_GPU_WEIGHT_ADDRESS_BOUNDED_WINDOW) == 0);
    CHECK(salt_gpu_weight_resource_pool_bind(SALT_GPU_RESOURCE_TRUNK, 0) == 0);
    CHECK(salt_gpu_weight_resource_pool_bind(SALT_GPU_RESOURCE_TRUNK, 0) != 0);            /* once */
    CHECK(salt_gpu_weight_window_bind(SALT_GPU_RESOURCE_TRUNK, 0, 0, 4096) != 0);          /* no windows into a pool */
    for (int i = 0; i < 8; i++) {
        const uint8_t *p = trunk_map + trunk[i].offset;
        const size_t elements = (size_t)trunk[i].rows * trunk[i].cols, vb = trunk[i].bits == 4 ? elements / 2 : elements;
        CHECK(salt_gpu_weight_resource_slot(SALT_GPU_RESOURCE_TRUNK, 0, p, (const uint32_t *)p, (const uint16_t *)(p + vb),
                                            (const uint16_t *)(p + vb + elements / 64 * 2), trunk[i].bits, trunk[i].rows,
                                            trunk[i].cols) == 0);
    }
    const int total_seats = layers * EXPERTS;
    CHECK(salt_cache_init_zerocopy(&cache, &pool, total_seats, 4) == 0);
    CHECK(salt_gpu_selected_resources_prepare(total_seats, total_seats) == 0);

    /* g4_init_device_residency: permanent spans, then one seat per expert of the pool */
    t0 = now_s();
    CHECK(open_residency(&model, (uint32_t)total_seats, 4, 1, &layout) == 0);
    t1 = now_s();
    CHECK(salt_gpu_residency_stats(&model.residency, &stats, sizeof stats) == 0);
    CHECK(layout.span_count == 2 && stats.permanent_spans == 2 && stats.permanent_bytes_populated <= layout.permanent_bytes);
    CHECK(stats.permanent_chunks >= 2 * ((layout.maximum_span_bytes + SLOT_BYTES - 1) / SLOT_BYTES) - 1);
    printf("residency-engine-path: permanent spans=%llu chunks=%llu bytes=%llu of a %llu-byte mapping, arena %.2f GB, %.3f s\n",
           (unsigned long long)stats.permanent_spans, (unsigned long long)stats.permanent_chunks,
           (unsigned long long)stats.permanent_bytes_populated, (unsigned long long)trunk_bytes,
           (double)model.residency.plan.device_budget_bytes / 1e9, t1 - t0);
    CHECK(salt_cache_set_resource_hooks(&cache, hook_fence, hook_bind, hook_unbind, &model) == 0);
    CHECK(salt_gpu_sync() == 0);
    CHECK(salt_gpu_weight_resource_usage(&usage, sizeof usage) == 0);
    CHECK(usage.device_copied_weight_bytes == stats.permanent_bytes_populated && usage.active_windows == 1);

    /* trunk projections from the permanent spans */
    for (int i = 0; i < 8; i++) {
        const uint8_t *p = trunk_map + trunk[i].offset;
        const size_t elements = (size_t)trunk[i].rows * trunk[i].cols, vb = trunk[i].bits == 4 ? elements / 2 : elements;
        const uint32_t *vals = (const uint32_t *)p;
        const uint16_t *scales = (const uint16_t *)(p + vb), *biases = (const uint16_t *)(p + vb + elements / 64 * 2);
        fill_x(x, trunk[i].cols);
        memset(got, 0xff, sizeof got);
        if (trunk[i].bits == 4) {
            salt_q4_matvec(vals, scales, biases, trunk[i].rows, trunk[i].cols, x, want);
            CHECK(salt_gpu_q4_matvec(vals, scales, biases, trunk[i].rows, trunk[i].cols, x, got) == 0);
        } else {
            salt_q8_matvec(vals, scales, biases, trunk[i].rows, trunk[i].cols, x, want);
            CHECK(salt_gpu_q8_matvec(vals, scales, biases, trunk[i].rows, trunk[i].cols, x, got) == 0);
        }
        CHECK(memcmp(got, want, sizeof(float) * (size_t)trunk[i].rows) == 0);
    }
    /* bytes of the mapping that no tensor occupies are not resident, and mapped-only mode refuses to copy them */
    {
        const uint8_t *p = trunk_map + trunk[3].offset + (size_t)EXPERTS * HIDDEN + (size_t)EXPERTS * HIDDEN / 64 * 4 + (1u << 20);
        CHECK(salt_gpu_q4_matvec((const uint32_t *)p, (const uint16_t *)(p + 4096), (const uint16_t *)(p + 8192), 8, 64, x, got) != 0);
    }

    /* phase 1: every expert of every layer takes a seat through the cache's bind hook */
    CHECK(salt_gpu_shared_buffer_alloc(&b.in, sizeof(float) * TOPK * HIDDEN) == 0);
    CHECK(salt_gpu_shared_buffer_alloc(&b.out, sizeof(float) * TOPK * HIDDEN) == 0);
    CHECK(salt_gpu_shared_buffer_alloc(&b.gate, sizeof(float) * TOPK * ROUTED) == 0);
    CHECK(salt_gpu_shared_buffer_alloc(&b.up, sizeof(float) * TOPK * ROUTED) == 0);
    {
        int experts[EXPERTS], slots[EXPERTS];
        for (int e = 0; e < EXPERTS; e++) experts[e] = e;
        t0 = now_s();
        for (int layer = 0; layer < layers; layer++) CHECK(salt_cache_getmany(&cache, layer, experts, EXPERTS, slots) >= 0);
        t1 = now_s();
    }
    CHECK(salt_gpu_residency_stats(&model.residency, &stats, sizeof stats) == 0);
    CHECK(model.binds == (uint64_t)total_seats && stats.population_completions == (uint64_t)total_seats &&
          stats.ready_slots == (uint32_t)total_seats && stats.active_leases == 0 && stats.backend_failures == 0);
    printf("residency-engine-path: seated %d experts (%.2f GB) in %.2f s = %.1f GB/s through the cache, ledger and staging\n",
           total_seats, (double)stats.population_bytes_completed / 1e9, t1 - t0,
           (double)stats.population_bytes_completed / 1e9 / (t1 - t0));
    for (int r = 0; r < 2; r++)
        for (int round = 0; round < 3; round++) {
            int experts[TOPK];
            for (int i = 0; i < TOPK; i++) experts[i] = (int)((7u + 16u * (unsigned)i + 5u * (unsigned)round) % EXPERTS);
            for (int i = 1; i < TOPK; i++)                                  /* ascending, as the router hands them over */
                for (int j = i; j > 0 && experts[j - 1] > experts[j]; j--) { int t = experts[j]; experts[j] = experts[j - 1]; experts[j - 1] = t; }
            fill_x(x, HIDDEN);
            CHECK(device_chain(&cache, &b, real_layers[r], experts, TOPK, x, "all seated") == 0);
        }
    {   /* a layer of holes: all-zero weights give all-zero outputs on both sides */
        int experts[TOPK] = {1, 2, 3, 5, 8, 13, 21, 34};
        if (layers > 3) CHECK(device_chain(&cache, &b, 1, experts, TOPK, x, "zero layer") == 0);
    }
    CHECK(model.binds == (uint64_t)total_seats && model.unbinds == 0);              /* nothing moved after seating */

    /* teardown of phase 1 the way the engine does it: the cache unbinds and retires every seat, then the ledger goes */
    salt_cache_free(&cache);
    CHECK(model.unbinds == (uint64_t)total_seats && model.fences >= 1);
    CHECK(salt_gpu_residency_stats(&model.residency, &stats, sizeof stats) == 0);
    CHECK(stats.retirements == (uint64_t)total_seats && stats.ready_slots == 0);
    CHECK(salt_gpu_residency_destroy(&model.residency) == 0);
    free(model.arena);
    model.arena = NULL;
    /* the permanent spans left with the arena: the trunk is no longer addressable */
    {
        const uint8_t *p = trunk_map + trunk[0].offset;
        const size_t vb = (size_t)DENSE * HIDDEN / 2;
        CHECK(salt_gpu_q4_matvec((const uint32_t *)p, (const uint16_t *)(p + vb), (const uint16_t *)(p + vb + (size_t)DENSE * HIDDEN / 32),
                                 DENSE, HIDDEN, x, got) != 0);
    }

    /* phase 2: sixteen seats, so the cache evicts; the spans are laid out and populated again */
    const int few = 16;
    memset(&model, 0, sizeof model);
    CHECK(salt_cache_init_zerocopy(&cache, &pool, few, 4) == 0);
    CHECK(salt_gpu_selected_resources_prepare(total_seats, total_seats) == 0);      /* the seat table stays as prepared */
    CHECK(open_residency(&model, few, 2, 1, &layout) == 0 && layout.span_count == 2);
    CHECK(salt_cache_set_resource_hooks(&cache, hook_fence, hook_bind, hook_unbind, &model) == 0);
    for (int round = 0; round < 12; round++) {
        int experts[TOPK];
        const int layer = real_layers[round & 1];
        for (int i = 0; i < TOPK; i++) experts[i] = (3 * round + 9 * i) % EXPERTS;
        for (int i = 1; i < TOPK; i++)
            for (int j = i; j > 0 && experts[j - 1] > experts[j]; j--) { int t = experts[j]; experts[j] = experts[j - 1]; experts[j - 1] = t; }
        fill_x(x, HIDDEN);
        CHECK(device_chain(&cache, &b, layer, experts, TOPK, x, "evicting") == 0);
    }
    CHECK(salt_gpu_residency_stats(&model.residency, &stats, sizeof stats) == 0);
    CHECK(model.unbinds > 0 && stats.retirements == model.unbinds && model.binds == model.unbinds + stats.ready_slots &&
          stats.peak_ready_slots <= (uint32_t)few && stats.backend_failures == 0);
    printf("residency-engine-path: %d seats: %llu populations, %llu evictions, results unchanged\n", few,
           (unsigned long long)model.binds, (unsigned long long)model.unbinds);
    {   /* the trunk answers again from the new spans */
        const uint8_t *p = trunk_map + trunk[4].offset;
        const size_t vb = (size_t)DENSE * HIDDEN / 2;
        fill_x(x, HIDDEN);
        salt_q4_matvec((const uint32_t *)p, (const uint16_t *)(p + vb), (const uint16_t *)(p + vb + (size_t)DENSE * HIDDEN / 32),
                       DENSE, HIDDEN, x, want);
        CHECK(salt_gpu_q4_matvec((const uint32_t *)p, (const uint16_t *)(p + vb), (const uint16_t *)(p + vb + (size_t)DENSE * HIDDEN / 32),
                                 DENSE, HIDDEN, x, got) == 0);
        CHECK(memcmp(got, want, sizeof(float) * DENSE) == 0);
    }

    salt_cache_free(&cache);
    CHECK(salt_gpu_residency_destroy(&model.residency) == 0);
    free(model.arena);

    /* phase 3: the ledger driven the way a prefetcher would: a fill is begun on every staging buffer before the
     * first is polled, so the engine's read of the next expert overlaps the copies of the previous ones (the cache's
     * bind hook of phases 1 and 2, like the model's, waits for each fill before it begins the next). */
    {
        const uint32_t seats = 512, staging = 8;
        const int layer = real_layers[0];
        uint64_t tickets[512];
        uint8_t *back = malloc(SLOT_BYTES);
        memset(&model, 0, sizeof model);
        CHECK(back && open_residency(&model, seats, staging, 0, &layout) == 0);
        t0 = now_s();
        for (uint32_t seat = 0; seat < seats; seat++) {
            SaltGpuResidencySource source;
            const int expert = (int)(seat % EXPERTS);
            const uint64_t logical = (uint64_t)layer * EXPERTS + (uint64_t)expert;
            const uint8_t *payload = salt_pool_expert_ptr(&pool, (size_t)layer * EXPERTS + (size_t)expert, SLOT_BYTES);
            CHECK(payload != NULL);
            if (seat >= staging) {                       /* the staging buffer about to be reused must be drained */
                const uint32_t old = seat - staging;
                int polled;
                do polled = salt_gpu_residency_population_poll(&model.residency, old, (uint64_t)layer * EXPERTS + old % EXPERTS,
                                                               old + 1u, tickets[old]);
                while (polled == 0);
                CHECK(polled == 1);
            }
            memset(&source, 0, sizeof source);
            source.resource.kind = SALT_GPU_RESOURCE_EXPERT_LAYER;
            source.resource.resource_id = (uint32_t)logical;
            source.logical_resource_id = logical;
            source.nbytes = SLOT_BYTES;
            source.read = payload_read;
            source.read_context = (void *)payload;
            CHECK(salt_gpu_residency_population_begin(&model.residency, seat, seat + 1u, &source, seat % staging,
                                                      &tickets[seat]) == 0);
        }
        for (uint32_t seat = seats - staging; seat < seats; seat++) {
            int polled;
            do polled = salt_gpu_residency_population_poll(&model.residency, seat, (uint64_t)layer * EXPERTS + seat % EXPERTS,
                                                           seat + 1u, tickets[seat]);
            while (polled == 0);
            CHECK(polled == 1);
        }
        t1 = now_s();
        printf("residency-engine-path: %u seats filled with %u fills in flight: %.1f GB/s\n", seats, staging,
               (double)seats * SLOT_BYTES / 1e9 / (t1 - t0));
        for (uint32_t seat = 0; seat < seats; seat += 37) {          /* the seats hold the experts' bytes */
            SaltGpuResidencyBinding binding;
            uintptr_t address = 0;
            CHECK(salt_gpu_residency_acquire(&model.residency, seat, (uint64_t)layer * EXPERTS + seat % EXPERTS, seat + 1u,
                                             &binding) == 1);
            CHECK(salt_gpu_residency_resolve(&model.residency, &binding, &address) == 0);
            CHECK(salt_mi355_dev_download(back, (const void *)address, SLOT_BYTES) == 0);
            CHECK(memcmp(back, salt_pool_expert_ptr(&pool, (size_t)layer * EXPERTS + seat % EXPERTS, SLOT_BYTES), SLOT_BYTES) == 0);
            CHECK(salt_gpu_residency_release(&model.residency, &binding) == 0);
        }
        CHECK(salt_gpu_residency_destroy(&model.residency) == 0);
        free(model.arena);
        free(back);
    }
    CHECK(salt_gpu_shared_buffer_free(&b.in) == 0 && salt_gpu_shared_buffer_free(&b.out) == 0);
    CHECK(salt_gpu_shared_buffer_free(&b.gate) == 0 && salt_gpu_shared_buffer_free(&b.up) == 0);
    CHECK(salt_gpu_weight_resource_deactivate(SALT_GPU_RESOURCE_TRUNK, 0) == 0);
    salt_gpu_set_mapped_only(0);
    CHECK(salt_pool_close(&pool) == 0);
    CHECK(salt_gpu_free() == 0);
    free(trunk_map);
    puts("residency-engine-path: PASS");
    return 0;
}
