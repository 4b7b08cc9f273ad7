// Affine-Q4 matvec for gfx950, bit-identical to the engine's CPU kernel.
//
// The arithmetic contract (reference src/kernels.c:220-250): per row, 32
// independent fp32 chains, chain j owning the columns c with c % 32 == j,
//     w = fl(fl(q * scale) + bias);  p = fl(w * x[c]);  acc[j] = fl(acc[j] + p)
// in ascending c, then the fixed fold  part[j] = sum_{a=0..7} acc[4a+j] from +0
// and y = (part0 + part2) + (part1 + part3).  Nothing may be reassociated, so
// parallelism comes from rows and from the 32 chains, never from splitting K.
//
// How the tiled kernel maps that to CDNA4:
//  * A workgroup owns a tile of 64 rows; lane l of every wave owns row l.
//    Wave t owns S of the 32 chains (S = 8, 4 or 2): the t-th S/2-byte slice
//    of every 16-byte block (32 columns) of the row.  Because the chain set is
//    wave-uniform, x[c] is a scalar (SGPR) operand fetched with s_load.
//  * 16 blocks (256 bytes per row, 16 KiB per tile) are staged per step into
//    LDS with coalesced 128-bit global loads, double-buffered; the row pitch
//    of 65 dwords makes every lane's slice read conflict-free.
//  * q -> float costs half an instruction: nibbles are isolated in bytes and
//    converted two at a time by v_cvt_pk_f32_fp8 (a byte 0..15 decodes to
//    q * 2^-9 exactly), with the power of two folded into the scale.  q*scale
//    is exact in fp32 (4-bit times 8-bit significand), so fma(q', scale', bias)
//    rounds once, exactly where the reference's separate add rounds.
//  * (scale', bias) pairs are converted once per tile step into LDS, not once
//    per wave.  A scale so large that scale * 2^9 would overflow flips the
//    tile to a path that multiplies and adds separately with the raw scale.
//  * The per-row fold runs in the documented order from LDS.
#include "device_math.h"
#include "mi355_internal.h"
#include "router_device.h"

#include <stddef.h>
#include <stdio.h>
#include <stdlib.h>

namespace mi355 {
namespace {

typedef float f32x2 __attribute__((ext_vector_type(2)));
// Activations are read-only for the lifetime of a launch and their address is
// wave-uniform, so they are read through the constant address space: the
// compiler then fetches them with scalar loads and feeds them to the VALU as
// SGPR operands.
typedef const float __attribute__((address_space(4))) *uniform_f32_ptr;
__device__ __forceinline__ uniform_f32_ptr as_uniform(const float *p) {
    return (uniform_f32_ptr)(uintptr_t)p;
}

constexpr int TILE_ROWS = 64;
constexpr int FOLD_PITCH = 33;
constexpr float BIG_SCALE = 0x1p118f;

__device__ __forceinline__ float bf16_to_f32(uint32_t half) { return __uint_as_float(half << 16); }

// Pointers that arrive inside a job record are generic; naming their address
// space lets the compiler use global_load / s_load instead of flat_load.
typedef const uint8_t __attribute__((address_space(1))) *global_u8_ptr;
typedef const uint16_t __attribute__((address_space(1))) *global_u16_ptr;
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
// 128-bit global loads need dword alignment only; the engine's expert pool file puts every tensor 8 bytes past a
// multiple of 16 (24-byte header), and those must still take the tiled path.
typedef u32x4 __attribute__((aligned(4))) u32x4_dword_aligned;
typedef const u32x4_dword_aligned __attribute__((address_space(1))) *global_u128_ptr;
typedef float __attribute__((address_space(1))) *global_f32_out_ptr;
typedef const uint64_t __attribute__((address_space(4))) *uniform_u64_ptr;

static_assert(sizeof(Q4Job) == 56 && offsetof(Q4Job, rows) == 40 && offsetof(Q4Job, tile0) == 44 &&
              offsetof(Q4Job, x_stride) == 48 && offsetof(Q4Job, y_stride) == 52,
              "find_job reads a job record as seven 64-bit words");

__device__ __forceinline__ Q4Job find_job(const Q4Launch &L, int tile) {
    if (L.njobs <= 1 && L.table == nullptr) return L.one;     // a table of one job (written on the device) is read like any other
    // 7 words per record, in a device table or inside the kernel arguments (the launch record is the kernel's only
    // argument, so the inline records sit at their offset in the kernarg segment)
    const uniform_u64_ptr words =
        L.table ? (uniform_u64_ptr)(uintptr_t)L.table
                : (uniform_u64_ptr)((const char __attribute__((address_space(4))) *)__builtin_amdgcn_kernarg_segment_ptr() +
                                    offsetof(Q4Launch, inline_jobs));
    int lo = 0, hi = L.njobs - 1;
    if (L.tiles_per_job > 0) {             // every job has the same number of tiles: no search
        lo = tile / L.tiles_per_job;
    } else {
        while (lo < hi) {                  // last job whose tile0 <= tile
            const int mid = (lo + hi + 1) >> 1;
            if ((int)(words[7 * mid + 5] >> 32) <= tile) lo = mid; else hi = mid - 1;
        }
    }
    const uniform_u64_ptr rec = words + 7 * lo;
    Q4Job job;
    job.vals = (const uint8_t *)rec[0];
    job.scales = (const uint8_t *)rec[1];
    job.biases = (const uint8_t *)rec[2];
    job.x = (const float *)rec[3];
    job.y = (float *)rec[4];
    job.rows = (int)(uint32_t)rec[5];
    job.tile0 = (int)(rec[5] >> 32);
    job.x_stride = (int)(uint32_t)rec[6];
    job.y_stride = (int)(rec[6] >> 32);
    return job;
}

// Eight nibbles of w as floats scaled by the converter's constant:
// q[n] = nibble_n * 2^-9 on gfx950.
__device__ __forceinline__ void nibbles_to_f32(uint32_t w, float (&q)[8]) {
    const uint32_t lo = w & 0x0F0F0F0Fu;
    const uint32_t hi = (w >> 4) & 0x0F0F0F0Fu;
    const f32x2 a = __builtin_amdgcn_cvt_pk_f32_fp8((int)lo, false);   // nibbles 0, 2
    const f32x2 b = __builtin_amdgcn_cvt_pk_f32_fp8((int)hi, false);   // nibbles 1, 3
    const f32x2 c = __builtin_amdgcn_cvt_pk_f32_fp8((int)lo, true);    // nibbles 4, 6
    const f32x2 d = __builtin_amdgcn_cvt_pk_f32_fp8((int)hi, true);    // nibbles 5, 7
    q[0] = a.x; q[1] = b.x; q[2] = a.y; q[3] = b.y;
    q[4] = c.x; q[5] = d.x; q[6] = c.y; q[7] = d.y;
}

// One packed word of a lane.  Nibble n belongs to block (first_block + n / S)
// of its scale group and to the lane's chain (n % S).  x holds the wave's
// activations in SGPRs: x[token][xbase + block * S + chain].
template <int S, int NB, int XN, int NNIB, bool SLOW>
__device__ __forceinline__ void consume_word(uint32_t w, int first_block, int xbase, float scale, float bias,
                                             const float (&x)[NB][XN], float code_scale, float (&acc)[NB][S]) {
    float q[8];
    nibbles_to_f32(w, q);
#pragma unroll
    for (int n = 0; n < NNIB; ++n) {
        const int blk = first_block + ((S == 8) ? 0 : n / S);
        const int ch = n % S;
        float wgt;
        if (!SLOW) {
            wgt = __builtin_fmaf(q[n], scale, bias);
        } else {
            const float qi = q[n] * code_scale;          // back to the integer value, exact
            wgt = qi * scale;
            wgt = wgt + bias;
        }
#pragma unroll
        for (int t = 0; t < NB; ++t) {
            const float xv = x[t][xbase + blk * S + ch];
            const float p = wgt * xv;
            acc[t][ch] = acc[t][ch] + p;
        }
    }
}

// How many 64-column groups of activations are fetched into SGPRs at once.
constexpr int x_batch_groups(int S, int NB) {
    const int fit = ((S == 8 || NB > 1) ? 32 : 64) / (2 * S * NB);     // SGPR budget for activations
    return fit >= 8 ? 8 : fit >= 4 ? 4 : fit >= 2 ? 2 : 1;
}

// CB = 32-column blocks staged per step.  16 keeps the tile's LDS small enough
// for three workgroups per compute unit; 32 is for launches with too few tiles
// to share a compute unit, where the amount of data in flight per workgroup is
// what hides the memory latency.
//
// PRO selects a prologue of the MoE decode step (0: none, jobs come from the
// launch): 1 = router top-k, the workgroup derives its gate or up job from the
// selection; 2 = the down projection of one selected expert, whose activations
// gelu_tanh(gate) * up are computed into LDS and reach the VALU in vector
// registers (every lane reads the same words) instead of through scalar loads;
// 3 = the same activation prologue for jobs of the launch (one token each).
template <int S, int NB, int CB, int PRO = 0>
__global__ __launch_bounds__((32 / S) * 64) void q4_tile_kernel(const Q4Launch L) {
    constexpr int CHUNK_BLOCKS = CB;
    constexpr int CHUNK_GROUPS = CB / 2;                   // 64-column scale groups per step
    constexpr int W_PITCH = 16 * CB + 4;                   // bytes per staged row: odd dword pitch
    constexpr int M_PITCH = 2 * CHUNK_GROUPS + 2;          // floats per staged row of (scale, bias)
    constexpr int W_STAGE = TILE_ROWS * W_PITCH;
    constexpr int M_STAGE = TILE_ROWS * M_PITCH;
    constexpr int WAVES = 32 / S;
    constexpr int THREADS = WAVES * 64;
    // A staging item is one scale group of one row: 32 bytes of codes (two blocks) and its (scale, bias).
    constexpr int ITEMS = (TILE_ROWS * CHUNK_GROUPS + THREADS - 1) / THREADS;
    constexpr int FOLD_BYTES = NB * TILE_ROWS * FOLD_PITCH * 4;
    constexpr int W_BYTES = 2 * W_STAGE > FOLD_BYTES ? 2 * W_STAGE : FOLD_BYTES;
    constexpr int XG = PRO >= 2 ? 2 : x_batch_groups(S, NB);        // LDS-fed activations sit in vector registers: short batches
    constexpr int XN = XG * 2 * S;
    static_assert(THREADS >= NB * TILE_ROWS, "fold needs one thread per (token, row)");

    __shared__ __attribute__((aligned(16))) uint8_t w_lds[W_BYTES];
    __shared__ __attribute__((aligned(16))) float m_lds[2 * M_STAGE];
    __shared__ __attribute__((aligned(16))) float x_lds[PRO >= 2 ? MOE_FUSE_MAX_ROUTED : 4];
    __shared__ int slow_flag;
    static_assert(PRO == 0 || NB == 1, "the MoE prologues serve the single-token kernel");
    static_assert(PRO != 1 || (sizeof(RouterShared) <= W_BYTES && THREADS >= MOE_FUSE_MAX_EXPERTS),
                  "the router prologue borrows the weight staging memory and one thread per expert");

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);

    Q4Job job;
    const float *act_gate = nullptr, *act_up = nullptr;     // PRO >= 2: the activation row is gelu_tanh(gate) * up
    if (PRO == 0) {
        job = find_job(L, blockIdx.x);
    } else if (PRO == 3) {
        // the job's activation row is gelu_tanh(gate) * up of the two rows its x names: x[i] and x[i + act_delta]
        job = find_job(L, blockIdx.x);
        act_gate = job.x; act_up = job.x + L.act_delta;
    } else {
        const MoeFuse &m = L.moe;
        const size_t n = (size_t)m.hidden * (size_t)m.routed;
        const size_t vals_bytes = n / 2, meta_bytes = (n / 64) * 2, proj_bytes = vals_bytes + 2 * meta_bytes;
        if (PRO == 1) {
            RouterShared &sh = *reinterpret_cast<RouterShared *>(w_lds);
            const bool publisher = (int)blockIdx.x == L.total_tiles;       // one workgroup past the tiles
            const int up_tiles = (m.routed + TILE_ROWS - 1) / TILE_ROWS;
            const int slot_index = (int)blockIdx.x / up_tiles;             // 2 * place + (0 gate | 1 up)
            const int place = slot_index >> 1, proj = slot_index & 1;
            int expert;
            if (!publisher && m.n_experts <= ROUTER_WAVE_MAX_EXPERTS) {
                // every wave finds the workgroup's expert on its own: no LDS, no barrier (the publisher keeps the
                // whole router: ordered sums, weights, status)
                expert = router_select_wave(m.logits, m.per_expert_scale, m.n_experts, m.topk, place);
                if (expert < 0) return;                                    // uniform: every wave sees the same inputs
            } else {
                router_topk_block(m.logits, m.per_expert_scale, m.n_experts, m.topk, true, publisher, sh);
                const int bad = sh.bad;
                if (publisher) {
                    if (tid == 0) *m.status = bad ? -1 : 0;
                    if (tid < m.topk && !bad) { m.selected[tid] = sh.out_sel[tid]; m.weights[tid] = sh.out_w[tid]; }
                    if (m.arrivals)                 // the down launch counts its workgroups per tile of the output
                        for (int i = tid; i < (m.hidden + TILE_ROWS - 1) / TILE_ROWS; i += THREADS) m.arrivals[i] = 0;
                    return;
                }
                if (bad) return;                                           // uniform
                expert = __builtin_amdgcn_readfirstlane(sh.out_sel[place]);
                __syncthreads();                                           // the staging memory is free again
            }
            job.vals = m.pool + (size_t)expert * m.expert_stride + (size_t)proj * proj_bytes;
            job.x = m.x;
            job.y = (proj ? m.up : m.gate) + (size_t)place * m.routed;
            job.rows = m.routed;
            job.tile0 = slot_index * up_tiles;
            job.x_stride = m.hidden;
            job.y_stride = m.routed;
        } else {
            if (*(const int __attribute__((address_space(4))) *)(uintptr_t)m.status != 0) return;
            const int down_tiles = (m.hidden + TILE_ROWS - 1) / TILE_ROWS;
            const int place = (int)blockIdx.x / down_tiles;
            const int expert = ((const int __attribute__((address_space(4))) *)(uintptr_t)m.selected)[place];
            act_gate = m.gate + (size_t)place * m.routed; act_up = m.up + (size_t)place * m.routed;
            job.vals = m.pool + (size_t)expert * m.expert_stride + 2 * proj_bytes;
            job.x = nullptr;
            job.y = m.expert_out + (size_t)place * m.hidden;
            job.rows = m.hidden;
            job.tile0 = place * down_tiles;
            job.x_stride = m.routed;
            job.y_stride = m.hidden;
        }
        job.scales = job.vals + vals_bytes;
        job.biases = job.scales + meta_bytes;
    }
    const int row0 = (blockIdx.x - job.tile0) * TILE_ROWS;
    const int R = job.rows;
    const int rows_here = R - row0 < TILE_ROWS ? R - row0 : TILE_ROWS;
    const int nblk = L.cols >> 5;
    const int ngrp = L.cols >> 6;
    const int nchunk = (nblk + CHUNK_BLOCKS - 1) / CHUNK_BLOCKS;
    const uint32_t row_bytes = (uint32_t)(L.cols >> 1);
    // wave-uniform bases of this tile; per-thread parts are 32-bit offsets
    const global_u8_ptr vals = (global_u8_ptr)(uintptr_t)job.vals + (size_t)row0 * row_bytes;
    const global_u16_ptr scales16 = (global_u16_ptr)(uintptr_t)job.scales + (size_t)row0 * ngrp;
    const global_u16_ptr biases16 =
        job.biases ? (global_u16_ptr)(uintptr_t)job.biases + (size_t)row0 * ngrp : (global_u16_ptr)0;
    const global_f32_out_ptr y = (global_f32_out_ptr)(uintptr_t)job.y;
    const uniform_f32_ptr xbase = as_uniform(job.x) + S * wave;

    // Per-thread staging geometry, fixed for the whole tile: item i of a thread
    // is group (tid % CHUNK_GROUPS) of row (tid / CHUNK_GROUPS + i * ROW_STEP), so
    // consecutive threads read consecutive 32-byte pieces of a row.  In LDS the
    // two blocks of a group are interleaved 16 bits at a time: dword t of the
    // group holds bytes 2t, 2t+1 of the first block and of the second, which is
    // exactly the pair of two-byte slices a four-chain wave consumes.
    constexpr int ROW_STEP = THREADS / CHUNK_GROUPS;
    const bool has_item = tid < TILE_ROWS * CHUNK_GROUPS;    // only narrower than the block when THREADS == 1024
    const uint32_t it_grp = tid % CHUNK_GROUPS;
    const uint32_t w_dst0 = ((tid / CHUNK_GROUPS) & (TILE_ROWS - 1)) * W_PITCH + it_grp * 32;
    const uint32_t m_dst0 = ((tid / CHUNK_GROUPS) & (TILE_ROWS - 1)) * M_PITCH + 2 * it_grp;
    uint32_t w_off[ITEMS], m_off[ITEMS];                     // source offsets of the item in step 0
#pragma unroll
    for (int i = 0; i < ITEMS; ++i) {
        const int row = ((tid / CHUNK_GROUPS) + i * ROW_STEP) & (TILE_ROWS - 1);
        const uint32_t rc = (uint32_t)(row < rows_here ? row : rows_here - 1);
        w_off[i] = rc * row_bytes + it_grp * 32;
        m_off[i] = rc * ngrp + it_grp;
    }

    u32x4 wreg[ITEMS][2];
    uint32_t sreg[ITEMS], breg[ITEMS];               // raw bf16 bits; nothing may consume them before commit

    // Loads of step ck into registers.  In every step but a partial last one
    // the address is a wave-uniform base plus the fixed per-thread offset; in
    // the last one group indices past the end of the row are clamped (the data
    // is staged but never consumed).
    // With several activation rows per launch the weights are fetched with the non-temporal policy: they are read
    // once, and keeping them out of the caches leaves the activations there (measured +17 % at four rows; at one row
    // the default policy is 1 % faster).
    auto load_weights = [](global_u8_ptr p) {
        return NB > 1 ? __builtin_nontemporal_load((global_u128_ptr)p) : *(global_u128_ptr)p;
    };
    auto issue = [&](int ck) {
        if (!has_item) return;
        const bool tail = (ck + 1) * CHUNK_GROUPS > ngrp;
        if (!tail) {
            const global_u8_ptr v = vals + (size_t)ck * (CHUNK_GROUPS * 32);
            const global_u16_ptr sp = scales16 + (size_t)ck * CHUNK_GROUPS;
            const global_u16_ptr bp = biases16 ? biases16 + (size_t)ck * CHUNK_GROUPS : (global_u16_ptr)0;
#pragma unroll
            for (int i = 0; i < ITEMS; ++i) {
                wreg[i][0] = load_weights(v + w_off[i]);
                wreg[i][1] = load_weights(v + w_off[i] + 16);
                sreg[i] = sp[m_off[i]];
                breg[i] = bp ? (uint32_t)bp[m_off[i]] : 0u;
            }
        } else {
#pragma unroll
            for (int i = 0; i < ITEMS; ++i) {
                int g = ck * CHUNK_GROUPS + (int)it_grp;
                const uint32_t back = g < ngrp ? 0u : (uint32_t)(g - (ngrp - 1));     // groups to step back to the last one
                const global_u8_ptr v = vals + (size_t)ck * (CHUNK_GROUPS * 32);
                wreg[i][0] = load_weights(v + (w_off[i] - back * 32));
                wreg[i][1] = load_weights(v + (w_off[i] - back * 32) + 16);
                const uint32_t at = m_off[i] + (uint32_t)ck * CHUNK_GROUPS - back;
                sreg[i] = scales16[at];
                breg[i] = biases16 ? (uint32_t)biases16[at] : 0u;
            }
        }
    };

    auto commit = [&](int stage) {
        if (!has_item) return;
#pragma unroll
        for (int i = 0; i < ITEMS; ++i) {
            uint32_t *dst = reinterpret_cast<uint32_t *>(w_lds + stage * W_STAGE + w_dst0 + i * ROW_STEP * W_PITCH);
            const uint32_t a[4] = {wreg[i][0].x, wreg[i][0].y, wreg[i][0].z, wreg[i][0].w};
            const uint32_t b[4] = {wreg[i][1].x, wreg[i][1].y, wreg[i][1].z, wreg[i][1].w};
#pragma unroll
            for (int d = 0; d < 4; ++d) {
                dst[2 * d] = __builtin_amdgcn_perm(b[d], a[d], 0x05040100u);          // low halves of a and b
                dst[2 * d + 1] = __builtin_amdgcn_perm(b[d], a[d], 0x07060302u);      // high halves
            }
            const float sc = bf16_to_f32(sreg[i]);
            const float bi = bf16_to_f32(breg[i]);
            if (!(__builtin_fabsf(sc) < BIG_SCALE)) slow_flag = 1;
            float *mdst = m_lds + stage * M_STAGE + m_dst0 + i * ROW_STEP * M_PITCH;
            mdst[0] = sc * L.code_scale;
            mdst[1] = bi;
        }
    };

    float acc[NB][S];
#pragma unroll
    for (int t = 0; t < NB; ++t)
#pragma unroll
        for (int c = 0; c < S; ++c) acc[t][c] = 0.0f;

    if (tid == 0) slow_flag = 0;
    issue(0);
    if (PRO >= 2) {
        // after the first weights have been sent for: they are on their way while the activation is computed
        for (int i = tid; i < L.cols; i += THREADS) x_lds[i] = det_gelu_tanh(act_gate[i]) * act_up[i];
    }
    __syncthreads();

    const int my_row = lane < rows_here ? lane : rows_here - 1;

    // x of `groups` consecutive scale groups starting at group g0 of the row
    auto load_x = [&](int g0, float (&xq)[NB][XN], int groups) {
        if (PRO >= 2) {                   // every lane reads the same LDS words: the activations travel in vector registers
            const float *xl = x_lds + g0 * 64 + S * wave;
#pragma unroll
            for (int k = 0; k < XN; ++k)
                if (k < groups * 2 * S) xq[0][k] = xl[(k / S) * 32 + (k % S)];
            return;
        }
        const uniform_f32_ptr xg = xbase + (size_t)g0 * 64;
#pragma unroll
        for (int t = 0; t < NB; ++t)
#pragma unroll
            for (int k = 0; k < XN; ++k)
                if (k < groups * 2 * S) xq[t][k] = xg[(size_t)t * job.x_stride + (k / S) * 32 + (k % S)];
    };

    for (int ck = 0; ck < nchunk; ++ck) {
        const int stage = ck & 1;
        const int remaining = ngrp - ck * CHUNK_GROUPS;
        const bool full = remaining >= CHUNK_GROUPS;
        const int gcount = full ? CHUNK_GROUPS : remaining;

        // The first batch of activations is requested before the barrier so
        // that its latency overlaps the staging writes and the wait.
        float xq[NB][XN];
        if (full) load_x(ck * CHUNK_GROUPS, xq, XG);

        commit(stage);
        __syncthreads();
        if (ck + 1 < nchunk) issue(ck + 1);

        const int slow = __builtin_amdgcn_readfirstlane(slow_flag);
        // wave t reads dword t (S == 4), dwords 2t and 2t+1 (S == 8) or dword t / 2 (S == 2) of every group
        const uint8_t *wrow = w_lds + stage * W_STAGE + lane * W_PITCH + (S == 2 ? (wave >> 1) * 4 : wave * S);
        const uint32_t byte_pick = 0x0C0C0000u | (uint32_t)((2 + (wave & 1)) << 8) | (uint32_t)(wave & 1);
        const float *mrow = m_lds + stage * M_STAGE + lane * M_PITCH;

        // LDS operands of group g of this step: the lane's nibbles and (scale', bias)
        auto fetch = [&](int g, uint32_t &w0, uint32_t &w1, float &scale, float &bias) {
            scale = mrow[2 * g];
            bias = mrow[2 * g + 1];
            w1 = 0;
            if (S == 8) {            // dwords 2t, 2t+1: (a01 b01), (a23 b23) -> the wave's four bytes of each block
                const uint32_t d0 = *reinterpret_cast<const uint32_t *>(wrow + g * 32);
                const uint32_t d1 = *reinterpret_cast<const uint32_t *>(wrow + g * 32 + 4);
                w0 = __builtin_amdgcn_perm(d1, d0, 0x05040100u);
                w1 = __builtin_amdgcn_perm(d1, d0, 0x07060302u);
            } else if (S == 4) {     // dword t: two bytes of the first block, two of the second
                w0 = *reinterpret_cast<const uint32_t *>(wrow + g * 32);
            } else {                 // S == 2: byte (t & 1) of each half of dword t / 2
                const uint32_t d = *reinterpret_cast<const uint32_t *>(wrow + g * 32);
                w0 = __builtin_amdgcn_perm(0u, d, byte_pick);
            }
        };

        if (full && !slow) {
            // Straight-line code over the eight groups of a full step.
#pragma unroll
            for (int batch = 0; batch < CHUNK_GROUPS / XG; ++batch) {
                if (batch > 0) load_x(ck * CHUNK_GROUPS + batch * XG, xq, XG);
#pragma unroll
                for (int gl = 0; gl < XG; ++gl) {
                    uint32_t w0, w1;
                    float scale, bias;
                    fetch(batch * XG + gl, w0, w1, scale, bias);
                    if (S == 8) {
                        consume_word<S, NB, XN, 8, false>(w0, 0, gl * 2 * S, scale, bias, xq, L.code_scale, acc);
                        consume_word<S, NB, XN, 8, false>(w1, 1, gl * 2 * S, scale, bias, xq, L.code_scale, acc);
                    } else {
                        consume_word<S, NB, XN, (S == 4 ? 8 : 4), false>(w0, 0, gl * 2 * S, scale, bias, xq,
                                                                                 L.code_scale, acc);
                    }
                }
            }
        } else {
            // Partial last step, or a tile that met an out-of-range scale:
            // whole activation batches first, then single groups.
            int g = 0;
            if (!slow) {
                for (; g + XG <= gcount; g += XG) {
                    load_x(ck * CHUNK_GROUPS + g, xq, XG);
#pragma unroll
                    for (int gl = 0; gl < XG; ++gl) {
                        uint32_t w0, w1;
                        float scale, bias;
                        fetch(g + gl, w0, w1, scale, bias);
                        if (S == 8) {
                            consume_word<S, NB, XN, 8, false>(w0, 0, gl * 2 * S, scale, bias, xq, L.code_scale, acc);
                            consume_word<S, NB, XN, 8, false>(w1, 1, gl * 2 * S, scale, bias, xq, L.code_scale, acc);
                        } else {
                            consume_word<S, NB, XN, (S == 4 ? 8 : 4), false>(w0, 0, gl * 2 * S, scale, bias, xq,
                                                                                     L.code_scale, acc);
                        }
                    }
                }
            }
            for (; g < gcount; ++g) {
                uint32_t w0, w1;
                float scale, bias;
                fetch(g, w0, w1, scale, bias);
                load_x(ck * CHUNK_GROUPS + g, xq, 1);
                if (slow) {
                    scale = bf16_to_f32(scales16[(uint32_t)my_row * ngrp + ck * CHUNK_GROUPS + g]);
                    if (S == 8) {
                        consume_word<S, NB, XN, 8, true>(w0, 0, 0, scale, bias, xq, L.code_scale, acc);
                        consume_word<S, NB, XN, 8, true>(w1, 1, 0, scale, bias, xq, L.code_scale, acc);
                    } else {
                        consume_word<S, NB, XN, (S == 4 ? 8 : 4), true>(w0, 0, 0, scale, bias, xq,
                                                                                L.code_scale, acc);
                    }
                } else {
                    if (S == 8) {
                        consume_word<S, NB, XN, 8, false>(w0, 0, 0, scale, bias, xq, L.code_scale, acc);
                        consume_word<S, NB, XN, 8, false>(w1, 1, 0, scale, bias, xq, L.code_scale, acc);
                    } else {
                        consume_word<S, NB, XN, (S == 4 ? 8 : 4), false>(w0, 0, 0, scale, bias, xq,
                                                                                 L.code_scale, acc);
                    }
                }
            }
        }
    }

    // Fold the 32 chains of each (token, row) in the reference's order.
    __syncthreads();
    float *fold = reinterpret_cast<float *>(w_lds);
#pragma unroll
    for (int t = 0; t < NB; ++t)
#pragma unroll
        for (int c = 0; c < S; ++c) fold[(t * TILE_ROWS + lane) * FOLD_PITCH + S * wave + c] = acc[t][c];
    __syncthreads();
    if (tid < NB * TILE_ROWS) {
        const int t = tid >> 6;
        const float *f = fold + (t * TILE_ROWS + lane) * FOLD_PITCH;
        float part[4] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int a = 0; a < 8; ++a)
#pragma unroll
            for (int j = 0; j < 4; ++j) part[j] = part[j] + f[4 * a + j];
        const float even = part[0] + part[2];
        const float odd = part[1] + part[3];
        if (PRO != 2 || !L.moe.arrivals) {
            if (lane < rows_here) y[(size_t)t * job.y_stride + row0 + lane] = even + odd;
        } else {                                        // uniform; NB == 1: these are the 64 lanes of wave 0
            // The layer output (reference gemma4_text.c:8301-8304: out = 0; out += o_i * w_i in ascending expert
            // order, product and sum rounded separately).  The topk workgroups that own these rows of the topk
            // experts count themselves in; the one that arrives last finds every expert's rows written and adds
            // them.  Which workgroup that is varies from run to run, the sum it forms does not.
            //
            // The rows travel as device-scope stores and loads (past the partition's cache, which other partitions
            // do not see), ordered by waiting for the stores before the count and for the count before the loads: a
            // fence would write the whole cache back, once per workgroup.
            const MoeFuse &m = L.moe;
            float *const mine = job.y + row0;                 // this expert's rows of expert_out
            if (lane < rows_here) __hip_atomic_store(mine + lane, even + odd, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            int before = 0;
            if (tid == 0) before = __hip_atomic_fetch_add(m.arrivals + (row0 / TILE_ROWS), 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            before = __builtin_amdgcn_readfirstlane(before);    // waits for the count's return
            if (before == m.topk - 1 && lane < rows_here) {
                float total = 0.0f;
                for (int e = 0; e < m.topk; ++e) {
                    const float o = __hip_atomic_load(m.expert_out + (size_t)e * m.hidden + row0 + lane, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    const float term = o * m.weights[e];
                    total = total + term;
                }
                m.out[row0 + lane] = total;
            }
        }
    }
}

// ---------------------------------------------------------------- generic
// Any column count and any byte alignment: lane = chain, 32 lanes per row, two
// rows per wave, byte loads.  Follows the flat element index k = r*C + c for
// the nibble and the scale group exactly as the reference does.
__device__ __forceinline__ uint32_t load_u16_bytes(global_u8_ptr p) { return (uint32_t)p[0] | ((uint32_t)p[1] << 8); }

template <int NB>
__global__ __launch_bounds__(256) void q4_generic_kernel(const Q4Launch L) {
    const Q4Job job = find_job(L, blockIdx.x);
    const int row0 = (blockIdx.x - job.tile0) * TILE_ROWS;
    const int chain = threadIdx.x & 31;
    const int sub = threadIdx.x >> 5;                    // 8 rows in flight per workgroup
    const int C = L.cols;
    const global_u8_ptr vals = (global_u8_ptr)(uintptr_t)job.vals;
    const global_u8_ptr scales = (global_u8_ptr)(uintptr_t)job.scales;
    const global_u8_ptr biases = (global_u8_ptr)(uintptr_t)job.biases;
    const float __attribute__((address_space(1))) *x = (const float __attribute__((address_space(1))) *)(uintptr_t)job.x;
    const global_f32_out_ptr y = (global_f32_out_ptr)(uintptr_t)job.y;
    for (int pass = 0; pass < TILE_ROWS / 8; ++pass) {
        const int row = row0 + pass * 8 + sub;
        const bool live = row < job.rows;
        const int r = live ? row : job.rows - 1;
        float acc[NB];
#pragma unroll
        for (int t = 0; t < NB; ++t) acc[t] = 0.0f;
        for (int c = chain; c < C; c += 32) {
            const size_t k = (size_t)r * (size_t)C + (size_t)c;
            const uint32_t byte = vals[k >> 1];
            const uint32_t q = (k & 1) ? (byte >> 4) : (byte & 15u);
            const size_t g = k >> 6;
            const float s = bf16_to_f32(load_u16_bytes(scales + 2 * g));
            const float b = biases ? bf16_to_f32(load_u16_bytes(biases + 2 * g)) : 0.0f;
            float wgt = (float)q * s;
            wgt = wgt + b;
#pragma unroll
            for (int t = 0; t < NB; ++t) {
                const float p = wgt * x[(size_t)t * job.x_stride + c];
                acc[t] = acc[t] + p;
            }
        }
        const int base = threadIdx.x & 32;               // first lane of this row's half-wave
#pragma unroll
        for (int t = 0; t < NB; ++t) {
            float part = 0.0f;
#pragma unroll
            for (int a = 0; a < 8; ++a) part = part + __shfl(acc[t], base + 4 * a + (chain & 3), 64);
            const float p0 = __shfl(part, base + 0, 64), p1 = __shfl(part, base + 1, 64);
            const float p2 = __shfl(part, base + 2, 64), p3 = __shfl(part, base + 3, 64);
            const float even = p0 + p2;
            const float odd = p1 + p3;
            if (live && chain == 0) y[(size_t)t * job.y_stride + row] = even + odd;
        }
    }
}

// Launches of at most this many tiles (one per compute unit) use the wide-step variant and two chains per lane.
constexpr int WIDE_TILE_LIMIT = 256;

template <int S>
int launch_tiles(const Q4Launch &L, hipStream_t stream) {
    const dim3 grid(L.total_tiles), block((32 / S) * 64);
    // One token with few tiles: a workgroup has its compute unit to itself and stages twice as much per step.
    if (L.tokens == 1 && S <= 4 && L.total_tiles <= WIDE_TILE_LIMIT) {
        note_kernel("q4_tile_kernel<%d,1,32,0>", S);
        hipLaunchKernelGGL((q4_tile_kernel<S, 1, 32>), grid, block, 0, stream, L);
        return hipGetLastError() == hipSuccess ? 0 : -1;
    }
    note_kernel("q4_tile_kernel<%d,%d,16,0>", S, L.tokens);
    switch (L.tokens) {
        case 1: hipLaunchKernelGGL((q4_tile_kernel<S, 1, 16>), grid, block, 0, stream, L); break;
        case 2: hipLaunchKernelGGL((q4_tile_kernel<S, 2, 16>), grid, block, 0, stream, L); break;
        case 3: hipLaunchKernelGGL((q4_tile_kernel<S, 3, 16>), grid, block, 0, stream, L); break;
        case 4: hipLaunchKernelGGL((q4_tile_kernel<S, 4, 16>), grid, block, 0, stream, L); break;
        default: return -1;
    }
    return hipGetLastError() == hipSuccess ? 0 : -1;
}

}  // namespace

bool q4_job_is_tileable(const Q4Job &job, int cols) {
    return cols >= 64 && (cols & 63) == 0 && ((uintptr_t)job.vals & 3) == 0 && ((uintptr_t)job.scales & 1) == 0 &&
           ((uintptr_t)job.biases & 1) == 0 && ((uintptr_t)job.x & 3) == 0 && ((uintptr_t)job.y & 3) == 0;
}

int q4_assign_tiles(Q4Job *table, int njobs) {
    int tiles = 0;
    for (int i = 0; i < njobs; ++i) {
        table[i].tile0 = tiles;
        tiles += (table[i].rows + TILE_ROWS - 1) / TILE_ROWS;
    }
    return tiles;
}

int q4_uniform_tiles(const Q4Job *table, int njobs) {
    const int first = (table[0].rows + TILE_ROWS - 1) / TILE_ROWS;
    for (int i = 1; i < njobs; ++i)
        if ((table[i].rows + TILE_ROWS - 1) / TILE_ROWS != first) return 0;
    return first;
}

int q4_moe_gate_up_launch(const Q4Launch &launch, hipStream_t stream) {
    Q4Launch L = launch;
    const MoeFuse &m = L.moe;
    if (m.n_experts < 1 || m.n_experts > MOE_FUSE_MAX_EXPERTS || m.topk < 1 || m.topk > m.n_experts ||
        m.topk > ROUTER_MAX_TOPK || m.hidden < 64 || (m.hidden & 63) || m.routed < 64 || (m.routed & 63))
        return -1;
    L.table = nullptr; L.njobs = 1; L.cols = m.hidden; L.tokens = 1;
    L.total_tiles = 2 * m.topk * ((m.routed + TILE_ROWS - 1) / TILE_ROWS);
    const dim3 grid(L.total_tiles + 1);                         // the extra workgroup publishes the router's outputs
    // measured at 176 tiles (eight experts of 704 rows): 1024-column steps 29.4 us per decode step, 512-column steps 29.1,
    // four chains per lane 30.4 and 33.4; the wide step is kept for launches that leave half the compute units idle
    if (L.total_tiles <= WIDE_TILE_LIMIT / 2)
        hipLaunchKernelGGL((q4_tile_kernel<2, 1, 32, 1>), grid, dim3(1024), 0, stream, L);
    else if (L.total_tiles <= WIDE_TILE_LIMIT)
        hipLaunchKernelGGL((q4_tile_kernel<2, 1, 16, 1>), grid, dim3(1024), 0, stream, L);
    else
        hipLaunchKernelGGL((q4_tile_kernel<4, 1, 16, 1>), grid, dim3(512), 0, stream, L);
    return hipGetLastError() == hipSuccess ? 0 : -1;
}

int q4_moe_down_launch(const Q4Launch &launch, hipStream_t stream) {
    Q4Launch L = launch;
    const MoeFuse &m = L.moe;
    if (m.topk < 1 || m.hidden < 64 || (m.hidden & 63) || m.routed < 64 || (m.routed & 63) ||
        m.routed > MOE_FUSE_MAX_ROUTED || (m.out == nullptr) != (m.arrivals == nullptr))
        return -1;
    L.table = nullptr; L.njobs = 1; L.cols = m.routed; L.tokens = 1;
    L.total_tiles = m.topk * ((m.hidden + TILE_ROWS - 1) / TILE_ROWS);
    const dim3 grid(L.total_tiles);
    // measured at 352 tiles (eight experts of 2816 rows): two chains per lane 31.4 us per decode step, four 29.4,
    // eight 31.4, wide steps 32.7 and 34.5
    if (L.total_tiles <= WIDE_TILE_LIMIT)
        hipLaunchKernelGGL((q4_tile_kernel<2, 1, 32, 2>), grid, dim3(1024), 0, stream, L);
    else
        hipLaunchKernelGGL((q4_tile_kernel<4, 1, 16, 2>), grid, dim3(512), 0, stream, L);
    return hipGetLastError() == hipSuccess ? 0 : -1;
}

int q4_activated_launch(const Q4Launch &L, hipStream_t stream) {
    if (L.total_tiles < 1 || L.tokens != 1 || L.cols < 64 || (L.cols & 63) || L.cols > MOE_FUSE_MAX_ROUTED) return -1;
    const dim3 grid(L.total_tiles);
    if (L.total_tiles <= WIDE_TILE_LIMIT)
        hipLaunchKernelGGL((q4_tile_kernel<2, 1, 32, 3>), grid, dim3(1024), 0, stream, L);
    else
        hipLaunchKernelGGL((q4_tile_kernel<4, 1, 16, 3>), grid, dim3(512), 0, stream, L);
    return hipGetLastError() == hipSuccess ? 0 : -1;
}

int q4_launch(const Q4Launch &L, int chains_per_lane, hipStream_t stream) {
    if (L.total_tiles < 1 || L.tokens < 1 || L.tokens > 4 || L.cols < 64 || (L.cols & 63)) return -1;
    int S = chains_per_lane;
    if (S == 0) {
        // Up to one tile per compute unit, sixteen waves per tile (two chains per lane) hide more of the LDS and
        // scalar-load latency; beyond that four chains per lane win (one token, 2816 columns: 12.4 against 15.5 us at
        // 256 tiles, 20.7 against 15.2 at 320, 23.3 against 17.6 at 512; eight chains per lane never do).
        S = L.total_tiles > WIDE_TILE_LIMIT ? 4 : 2;
    }
    switch (S) {
        case 8: return launch_tiles<8>(L, stream);
        case 4: return launch_tiles<4>(L, stream);
        case 2: return launch_tiles<2>(L, stream);
        default: return -1;
    }
}

int q4_launch_generic(const Q4Launch &L, hipStream_t stream) {
    if (L.total_tiles < 1 || L.tokens < 1 || L.tokens > 4 || L.cols < 1) return -1;
    const dim3 grid(L.total_tiles), block(256);
    switch (L.tokens) {
        case 1: hipLaunchKernelGGL((q4_generic_kernel<1>), grid, block, 0, stream, L); break;
        case 2: hipLaunchKernelGGL((q4_generic_kernel<2>), grid, block, 0, stream, L); break;
        case 3: hipLaunchKernelGGL((q4_generic_kernel<3>), grid, block, 0, stream, L); break;
        case 4: hipLaunchKernelGGL((q4_generic_kernel<4>), grid, block, 0, stream, L); break;
        default: return -1;
    }
    return hipGetLastError() == hipSuccess ? 0 : -1;
}

// ---------------------------------------------------------------- converter probe
namespace {
__global__ void probe_converters_kernel(float *fp8_values, float *fp4_values) {
    const uint32_t byte = threadIdx.x;                   // 256 threads
    const f32x2 a = __builtin_amdgcn_cvt_pk_f32_fp8((int)byte, false);
    fp8_values[byte] = a.x;
    const f32x2 b = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(byte, 1.0f, 0);
    fp4_values[2 * byte] = b.x;                          // low nibble
    fp4_values[2 * byte + 1] = b.y;                      // high nibble
}
}  // namespace

namespace {
__global__ __launch_bounds__(256) void clear_words_kernel(uint32_t *dst, size_t words) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i < words) dst[i] = 0u;
}
__global__ __launch_bounds__(256) void copy_words_kernel(uint32_t *dst, const uint32_t *src, size_t words) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i < words) dst[i] = src[i];
}
}  // namespace

// Word copy by a kernel, for sources the device can address (mapped pinned host memory included): for a few
// kilobytes a launch is cheaper than a copy command.
int copy_words_launch(void *dst, const void *src, size_t words, hipStream_t stream) {
    if (words == 0) return 0;
    hipLaunchKernelGGL(copy_words_kernel, dim3((unsigned)((words + 255) / 256)), dim3(256), 0, stream, (uint32_t *)dst,
                       (const uint32_t *)src, words);
    return hipGetLastError() == hipSuccess ? 0 : -1;
}

// Zero fill by a kernel: a memset node recorded into a caller's graph capture is not reliable on replay here.
int clear_words_launch(void *dst, size_t words, hipStream_t stream) {
    if (words == 0) return 0;
    hipLaunchKernelGGL(clear_words_kernel, dim3((unsigned)((words + 255) / 256)), dim3(256), 0, stream, (uint32_t *)dst,
                       words);
    return hipGetLastError() == hipSuccess ? 0 : -1;
}

int probe_converters_launch(float *fp8_values, float *fp4_values, hipStream_t stream) {
    hipLaunchKernelGGL(probe_converters_kernel, dim3(1), dim3(256), 0, stream, fp8_values, fp4_values);
    return hipGetLastError() == hipSuccess ? 0 : -1;
}

}  // namespace mi355
