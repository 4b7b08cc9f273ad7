/* Drives the reference's own PUBLIC functions through one MoE layer, for the CPU-baseline leg of the benchmark and
 * as a second statement of the step for the checker's tests.  This file is this repository's; it is compiled into
 * oracle/_ref/libsaltref.so beside the reference sources it calls (oracle/Makefile `ref`) and is test
 * infrastructure like everything else under oracle/.
 *
 * The reference's decode step lives in static functions of its model file (expert_worker, routed_experts:
 * models/gemma4-26b-a4b/src/gemma4_text.c:7608-7649, 7908-8306); what they call is public and is called here in the
 * same order: salt_gemma4_router_topk, the ascending sort (:7923-7930), per expert salt_q4_matvec (gate, up),
 * salt_gemma4_gelu_tanh, salt_q4_matvec (down) inside the expert scope (salt_kernels_set_in_expert: no row split
 * inside an expert), experts spread over min(cores, 8) threads (:8247-8277), then the ordered weighted sum
 * (:8301-8304).  The grouped prefill is salt_moe_group_execute itself (src/moe_group.c:9) with callbacks that run an
 * expert over its rows with salt_q4_matvec_batch, as g4_group_run does (gemma4_text.c:8749-8860). */
#include <pthread.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#include "salt/kernels.h"
#include "salt/moe_group.h"

float salt_gemma4_gelu_tanh(float x);
int salt_gemma4_router_topk(const float *logits, const float *per_expert_scale, int n_experts, int topk, int *selected,
                            float *weights);

typedef struct {
    const uint8_t *pool;
    size_t stride;
    int hidden, routed;
} RefPool;

static size_t proj_bytes(const RefPool *p) {
    const size_t n = (size_t)p->hidden * (size_t)p->routed;
    return n / 2 + 2 * ((n / 64) * 2);
}

static void expert_rows(const RefPool *p, int expert, int rows, const float *in, float *gate, float *up, float *out) {
    const size_t n = (size_t)p->hidden * (size_t)p->routed, vals = n / 2, meta = (n / 64) * 2, proj = proj_bytes(p);
    const uint8_t *slot = p->pool + (size_t)expert * p->stride;
    const uint8_t *g = slot, *u = slot + proj, *d = slot + 2 * proj;
    if (rows == 1) {
        salt_q4_matvec((const uint32_t *)g, (const uint16_t *)(g + vals), (const uint16_t *)(g + vals + meta), p->routed,
                       p->hidden, in, gate);
        salt_q4_matvec((const uint32_t *)u, (const uint16_t *)(u + vals), (const uint16_t *)(u + vals + meta), p->routed,
                       p->hidden, in, up);
    } else {
        salt_q4_matvec_batch((const uint32_t *)g, (const uint16_t *)(g + vals), (const uint16_t *)(g + vals + meta),
                             p->routed, p->hidden, rows, in, gate);
        salt_q4_matvec_batch((const uint32_t *)u, (const uint16_t *)(u + vals), (const uint16_t *)(u + vals + meta),
                             p->routed, p->hidden, rows, in, up);
    }
    for (size_t i = 0; i < (size_t)rows * (size_t)p->routed; i++) gate[i] = salt_gemma4_gelu_tanh(gate[i]) * up[i];
    if (rows == 1)
        salt_q4_matvec((const uint32_t *)d, (const uint16_t *)(d + vals), (const uint16_t *)(d + vals + meta), p->hidden,
                       p->routed, gate, out);
    else
        salt_q4_matvec_batch((const uint32_t *)d, (const uint16_t *)(d + vals), (const uint16_t *)(d + vals + meta),
                             p->hidden, p->routed, rows, gate, out);
}

typedef struct {
    const RefPool *pool;
    const int *selected;
    const float *x;
    float *gate, *up, *expert_out;
    int first, stride, topk;
} DecodeWorker;

static void *decode_worker(void *opaque) {
    DecodeWorker *w = (DecodeWorker *)opaque;
    for (int i = w->first; i < w->topk; i += w->stride)
        expert_rows(w->pool, w->selected[i], 1, w->x, w->gate + (size_t)i * w->pool->routed,
                    w->up + (size_t)i * w->pool->routed, w->expert_out + (size_t)i * w->pool->hidden);
    return NULL;
}

/* scratch: topk * (2 * routed + hidden) floats.  0 ok, -1 as the reference's router. */
int refdrv_moe_decode_step(const uint8_t *pool, size_t stride, int n_experts, int topk, int hidden, int routed,
                           const float *logits, const float *per_expert_scale, const float *x, int *selected,
                           float *weights, float *expert_out, float *out, float *scratch, int threads) {
    if (topk < 1 || topk > 64) return -1;
    if (salt_gemma4_router_topk(logits, per_expert_scale, n_experts, topk, selected, weights) != 0) return -1;
    for (int i = 0; i < topk; i++)            /* gemma4_text.c:7923-7930 */
        for (int j = i + 1; j < topk; j++)
            if (selected[j] < selected[i]) {
                const int e = selected[i]; selected[i] = selected[j]; selected[j] = e;
                const float v = weights[i]; weights[i] = weights[j]; weights[j] = v;
            }
    const RefPool p = {pool, stride, hidden, routed};
    float *gate = scratch, *up = scratch + (size_t)topk * routed;
    float *eo = expert_out ? expert_out : scratch + (size_t)2 * topk * routed;
    if (threads > topk) threads = topk;
    if (threads < 1) threads = 1;
    const int prior = salt_kernels_in_expert();
    salt_kernels_set_in_expert(1);
    pthread_t tid[64];
    DecodeWorker work[64];
    for (int t = 0; t < threads; t++) {
        work[t] = (DecodeWorker){&p, selected, x, gate, up, eo, t, threads, topk};
        if (t + 1 < threads && pthread_create(&tid[t], NULL, decode_worker, &work[t]) != 0) {
            salt_kernels_set_in_expert(prior);
            return -1;
        }
    }
    decode_worker(&work[threads - 1]);
    for (int t = 0; t + 1 < threads; t++) pthread_join(tid[t], NULL);
    salt_kernels_set_in_expert(prior);
    for (int d = 0; d < hidden; d++) {         /* gemma4_text.c:8301-8304 */
        float sum = 0.0f;
        for (int i = 0; i < topk; i++) sum += eo[(size_t)i * hidden + d] * weights[i];
        out[d] = sum;
    }
    return 0;
}

typedef struct {
    RefPool pool;
    float *gate, *up;      /* [rows capacity][routed] */
} GroupContext;

static int group_acquire(void *context, int expert, void **lease) {
    (void)context;
    *lease = (void *)(intptr_t)(expert + 1);
    return 0;
}
static int group_release(void *context, int expert, void *lease) {
    (void)context; (void)expert; (void)lease;
    return 0;
}
static int group_run(void *context, int expert, void *lease, int group, const float *inputs, float *outputs) {
    GroupContext *c = (GroupContext *)context;
    (void)lease;
    expert_rows(&c->pool, expert, group, inputs, c->gate, c->up, outputs);
    return 0;
}

/* The reference's grouped executor over `tokens` tokens.  scratch: tokens * (2 * routed + 2 * hidden + topk * hidden)
 * floats (expert intermediates, then the executor's own fixed-address scratch, moe_group.h:8-24). */
int refdrv_moe_group(const uint8_t *pool, size_t stride, int n_experts, int topk, int hidden, int routed, int tokens,
                     const int *selected, const float *weights, const float *inputs, float *outputs, float *scratch) {
    if (n_experts < 1 || n_experts > 4096 || tokens < 1) return -1;
    GroupContext context = {{pool, stride, hidden, routed}, scratch, scratch + (size_t)tokens * routed};
    unsigned char used[4096], acquired[4096];
    void *leases[4096];
    int expert_ids[4096];
    SaltMoEGroupScratch fixed;
    memset(&fixed, 0, sizeof fixed);
    fixed.used = used; fixed.acquired = acquired; fixed.leases = leases; fixed.expert_ids = expert_ids;
    fixed.group_inputs = scratch + (size_t)2 * tokens * routed;
    fixed.group_outputs = fixed.group_inputs + (size_t)tokens * hidden;
    fixed.selection_outputs = fixed.group_outputs + (size_t)tokens * hidden;
    fixed.expert_capacity = 4096;
    fixed.group_element_capacity = (size_t)tokens * hidden;
    fixed.selection_element_capacity = (size_t)tokens * topk * hidden;
    SaltMoEGroupJob job;
    memset(&job, 0, sizeof job);
    job.batch = tokens; job.topk = topk; job.n_experts = n_experts; job.hidden = hidden;
    job.selected = selected; job.weights = weights; job.inputs = inputs; job.outputs = outputs;
    job.scratch = &fixed;
    SaltMoEGroupOps ops;
    memset(&ops, 0, sizeof ops);
    ops.acquire = group_acquire; ops.run = group_run; ops.release = group_release;
    return salt_moe_group_execute(&job, &ops, &context);
}
