// Internal declarations shared by the kernel translation units and the C ABI.
#pragma once

#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

namespace mi355 {

// Name and template arguments of the matvec kernel launched last (diagnostics: salt_mi355_last_kernel).
void note_kernel(const char *format, ...) __attribute__((format(printf, 1, 2)));

// ---------------------------------------------------------------- affine Q4

// One weight matrix against `tokens` activation rows.  All pointers are
// device pointers.  Rows are processed in tiles of 64; tile0 is the index of
// the job's first tile inside the launch that carries it.
struct Q4Job {
    const uint8_t *vals;      // packed nibbles, row-major, C/2 bytes per row
    const uint8_t *scales;    // bf16 per 64 elements
    const uint8_t *biases;    // bf16 per 64 elements, may be null (bias 0)
    const float *x;           // [tokens][x_stride]
    float *y;                 // [tokens][y_stride]
    int rows;
    int tile0;
    int x_stride;
    int y_stride;
};

// The MoE decode step folded into two launches of the tile kernel: the gate/up launch runs the router in its
// prologue (every workgroup finds its own expert; one extra workgroup publishes selection, weights and status), the
// down launch computes gelu_tanh(gate) * up of its expert into LDS and reads its activations from there.
struct MoeFuse {
    const float *logits, *per_expert_scale;
    const uint8_t *pool;
    size_t expert_stride;
    const float *x;               // [hidden]
    float *gate, *up;             // [topk][routed]
    float *act;                   // [topk][routed]: gelu_tanh(gate) * up (the two-launch plan of moe_dot16.hip)
    float *expert_out;            // [topk][hidden]
    int *selected;                // [topk], ascending expert id
    float *weights;               // [topk]
    int *status;                  // 0, or -1 when the router rejected its input (then nothing else is written)
    int n_experts, topk, hidden, routed;
    // q4_moe_gate_up_launch / q4_moe_down_launch only, both null or both set: the down launch also writes the layer
    // output.  arrivals holds one counter per 64-row tile of the output; the gate/up launch zeroes them, and the last
    // of the topk workgroups of the down launch to finish a tile adds that tile's expert outputs in expert order.
    float *out;                   // [hidden]
    int *arrivals;                // [ceil(hidden / 64)]
};
constexpr int MOE_FUSE_MAX_ROUTED = 4096;      // activations of one expert held in LDS by the down launch
constexpr int MOE_FUSE_MAX_EXPERTS = 512;      // one thread per expert in the gate/up prologue

constexpr int Q4_INLINE_JOBS = 16;

struct Q4Launch {
    Q4Job one;                // used when njobs == 1
    const Q4Job *table;       // device array of njobs jobs sorted by tile0; nullptr: the jobs travel in `inline_jobs`
    int njobs;
    int cols;                 // C, shared by every job of the launch
    int tokens;               // 1..4 activation rows per job
    int total_tiles;
    float code_scale;         // 1 / (value the fp8 converter gives byte 1)
    int tiles_per_job;        // > 0 when every job of the table has this many tiles (tile -> job by division), else 0
    MoeFuse moe;              // only read by q4_moe_gate_up_launch / q4_moe_down_launch
    long long act_delta;      // q4_activated_launch: floats from a job's gate row (its x) to its up row
    // Up to Q4_INLINE_JOBS job records inside the kernel arguments: a decode-sized batch (the gate and up projections
    // of eight experts) then needs no table upload.  Must stay the last member.
    Q4Job inline_jobs[Q4_INLINE_JOBS];
};
int q4_moe_gate_up_launch(const Q4Launch &launch, hipStream_t stream);   // fills tiles and jobs from launch.moe
int q4_moe_down_launch(const Q4Launch &launch, hipStream_t stream);

// chains_per_lane: 8, 4 or 2; 0 lets the launcher choose from the tile count.
int q4_launch(const Q4Launch &launch, int chains_per_lane, hipStream_t stream);
// Any C, any byte alignment: one wave64 computes two rows, lane = chain.
int q4_launch_generic(const Q4Launch &launch, hipStream_t stream);
// One token per job; a job's activations are gelu_tanh(x[i]) * x[i + act_delta], computed in every workgroup's
// prologue (cols <= MOE_FUSE_MAX_ROUTED, tileable jobs).
int q4_activated_launch(const Q4Launch &launch, hipStream_t stream);
// true when every pointer and the column count meet the tiled kernel's needs
bool q4_job_is_tileable(const Q4Job &job, int cols);

// fills table[i].tile0 and returns the launch's tile count
int q4_assign_tiles(Q4Job *table, int njobs);
// the common tile count of the jobs, or 0 when they differ
int q4_uniform_tiles(const Q4Job *table, int njobs);

// ---------------------------------------------------------------- affine Q4 decode matvec, tolerance class
// (q4_dot.hip): per scale group  scale * sum q*x + bias * sum x  with the integer dot products exact.

constexpr int DOT_BLOCK_ROWS = 32;         // rows per block; a wave walks whole blocks
constexpr int DOT_MIN_COLS = 512;          // the streaming kernel takes 512 .. 8192 columns in multiples of 64;
constexpr int DOT_MAX_COLS = 8192;         // callers send everything else to the exact kernel
constexpr int DOT_LDS_LIMIT = 160 * 1024;

// How a launch is cut: waves per workgroup, steps of LDS per wave, parts a row is cut into along its columns
// (ksplit waves share one block of 32 rows), consecutive blocks a wave walks back to back (1 or 2).  A workgroup owns
// waves / ksplit * blocks_per_wave blocks.
struct DotShape { int waves, stages, ksplit, blocks_per_wave; };

struct Q4DotLaunch {
    Q4Job one;                // used when table == nullptr; tile0 = index of the job's first workgroup
    const Q4Job *table;       // device array of njobs jobs sorted by tile0
    int njobs;
    int cols;
    int tokens;               // 1..4, at most q4_dot_tokens_per_pass(cols)
    int total_wgs;
    int ksplit;               // filled by q4_dot_launch from the shape
    int wgs_per_job;          // > 0 when every job of the table has this many workgroups (workgroup -> job by division)
    // q4_dot16_launch only.  passes > 1: the launch covers tokens_total tokens in passes of `tokens` each (the last
    // may hold fewer); every block of rows is walked once per pass by workgroups that the dispatcher places next
    // to each other, so that all passes but the first find the weights in the cache they share.
    int passes, tokens_total;
    int windows;              // q4_dot16_launch only.  2: every row is walked in two column windows (q4_dot16_window_waves)
    MoeFuse moe;              // only read by q4_dot_moe_gate_up_launch / q4_dot_moe_down_launch
    // Up to Q4_INLINE_JOBS job records inside the kernel arguments (table == nullptr, njobs > 1): a decode-sized
    // batch then needs no table upload.  Must stay the last member.
    Q4Job inline_jobs[Q4_INLINE_JOBS];
};
bool q4_dot_takes(int cols);
int q4_dot_tokens_per_pass(int cols);      // 0: the column count does not fit at all
DotShape q4_dot_shape(int cols, int tokens, long long total_blocks);
int q4_dot_launch(const Q4DotLaunch &launch, const DotShape &shape, hipStream_t stream);
// The same arithmetic on blocks of sixteen rows (q4_dot16.hip): one or two tokens, launches with many blocks.
// q4_dot16_waves: waves per workgroup to use (a workgroup owns that many blocks of 16 rows), or 0 = use the 32-row kernel.
int q4_dot16_waves(int cols, int tokens, long long total_blocks32);
int q4_dot16_launch(const Q4DotLaunch &launch, int waves, hipStream_t stream);
bool q4_dot16_takes_passes(int tokens_per_pass, int waves);
// Waves per workgroup when rows too wide for all tokens' digit planes are walked in two column windows (launch.windows
// = 2, three or four tokens), or 0 when that shape does not serve the launch.
int q4_dot16_window_waves(int cols, int tokens, long long total_blocks32);
// The MoE decode step's two matvec launches on the streaming kernel (router top-k in the prologue of the first,
// gelu_tanh(gate) * up in the prologue of the second); -1: the geometry is not served.
// The whole step in two launches (moe_dot16.hip): gate + up + activation, then down + ordered weighted sum; `out`
// receives the layer output, moe.expert_out (optional) the expert outputs.  -1: the geometry is not served.
int moe_static_scratch_prepare();      // backend_dev.hip: looks up the static MoE workspace of the current device
constexpr int MOE16_NOT_SERVED = 1;
int moe16_step_launch(const MoeFuse &moe, float *out, hipStream_t stream);
bool q4_dot_moe_serves(const MoeFuse &moe);
int q4_dot_moe_gate_up_launch(const MoeFuse &moe, hipStream_t stream);
int q4_dot_moe_down_launch(const MoeFuse &moe, hipStream_t stream);

// ---------------------------------------------------------------- affine Q4 on MFMA (tolerance class)

// One weight matrix against `tokens` activation rows that have been split
// into three bf16 planes (x = hi + mid + lo) with per-64-column sums.
constexpr int MFMA_TM = 64;   // tokens per workgroup of the matrix-core kernel; its weight rows: mfma_tile_rows()

struct MfmaJob {
    const uint8_t *vals, *scales, *biases;   // biases may be null
    const uint16_t *planes;   // plane 0 of this job's first token; plane p lies p * plane_stride elements further
    const float *xsum;        // [tokens][C/64]
    float *y;                 // [tokens][rows]
    int tokens;
    int rows;
    int tile0;
    int row_base;             // with a row map: index of this job's first token in the map
};

struct MfmaLaunch {
    MfmaJob one;
    const MfmaJob *table;
    int njobs;
    int cols;
    int total_tiles;          // grid size; an upper bound when the counts below live on the device
    size_t plane_stride;      // elements between planes
    const int *njobs_dev;     // optional: job and tile counts produced by an earlier kernel;
    const int *total_tiles_dev;   // workgroups past *total_tiles_dev exit at once
    const int *row_map;       // optional gather: token t of a job reads plane row row_map[row_base + t] / map_divisor
    int map_divisor;
    int blocks_per_wave;      // the tile is 64 tokens x 64 * blocks_per_wave rows (mfma_blocks_per_wave()); 0 = choose (single job only)
};

int q4_mfma_launch(const MfmaLaunch &launch, hipStream_t stream);
int mfma_tile_rows(int blocks_per_wave);
int mfma_tiles(int tokens, int rows, int blocks_per_wave);
int mfma_blocks_per_wave(long long wide_tiles);
// rows of fp32 -> bf16 planes + group sums; output row r reads input row row_map[r] / map_divisor when a map is
// given; with a gate the value split is gelu_tanh(gate) * x (gate has the layout of x)
int x_split_launch(const float *x, const float *gate, const int *row_map, int map_divisor, int x_stride, int rows,
                   int cols, uint16_t *planes, size_t plane_stride, float *xsum, hipStream_t stream);

// ---------------------------------------------------------------- NVFP4

struct Fp4Job {
    const uint8_t *packed;    // E2M1 codes, two per byte, C/2 bytes per row
    const uint8_t *scales;    // E4M3FN, one per 16 columns
    const float *x;           // [tokens][x_stride] activation used as given
    float *y;                 // [tokens][rows]
    float weight_global_scale;  // 1 / stored divisor
    int rows;
    int tile0;
    int x_stride;
};

struct Fp4Launch {
    Fp4Job one;
    const Fp4Job *table;
    int njobs;
    int cols;
    int tokens;
    int total_tiles;
    // Fused activation pass (single job, one token, cols <= FP4_FUSED_MAX_COLS): x is the raw activation, every
    // workgroup quantises and dequantises it into LDS, *status (cleared by the caller) becomes -1 for a non-finite
    // activation, and nothing is published then.
    int qdq;
    float input_global_scale;
    int *status;
};
constexpr int FP4_FUSED_MAX_COLS = 8192;

int fp4_launch(const Fp4Launch &launch, int chains_per_lane, hipStream_t stream);

// The reference matvec (activation quantised inside the launch) on the tolerance-class streaming kernel
// (nvfp4_dot.hip).  tile0 of a job = index of its first workgroup; job.x is the raw activation.
struct Fp4DotLaunch {
    Fp4Job one;
    const Fp4Job *table;
    int njobs;
    int cols;
    int tokens;               // 1..4
    int total_wgs;
    int ksplit;               // filled by fp4_dot_launch from the shape
    int wgs_per_job;          // > 0 when every job of the table has this many workgroups
    float input_global_scale;
    int *status;              // cleared by the caller; becomes -1 when an activation is not finite
};
bool fp4_dot_takes(int cols);
DotShape fp4_dot_shape(int cols, int tokens, long long total_blocks);
int fp4_dot_launch(const Fp4DotLaunch &launch, const DotShape &shape, hipStream_t stream);
// activation quantise/dequantise per 16-block; any of packed/scales/dequant/plane may be null.  plane receives
// code value * block scale as bf16 (exact), the activation operand of the matrix-core matmul.
int fp4_qdq_launch(const float *input, int cols, int tokens, float input_global_scale,
                   uint8_t *packed, uint8_t *scales, float *dequant, uint16_t *plane, int *status,
                   hipStream_t stream);
// The same pass reporting per workgroup instead of through one word that somebody must have cleared: flags[i]
// receives 0 or -1 from workgroup i, every one of the fp4_qdq_flag_count(cols, tokens) words is written.
int fp4_qdq_flag_count(int cols, int tokens);
int fp4_qdq_flags_launch(const float *input, int cols, int tokens, float input_global_scale, uint16_t *plane,
                         int *flags, hipStream_t stream);

// Prefill-sized NVFP4 matmul on the matrix cores (tolerance class): ys[token][row] =
// out_scale * sum_c (code * block scale)[row][c] * plane[token][c].
struct Fp4MfmaLaunch {
    const uint8_t *packed, *scales;
    const uint16_t *plane;    // [tokens][cols] bf16
    float *ys;                // [tokens][rows]
    float *partials;          // [ksplit][tokens][rows], used when ksplit > 1
    const int *status;        // nothing is published unless *status == 0 ...
    // ... or, when flags is set, unless all nflags words are 0; the launch then writes the outcome (0 or -1) to
    // outcome and, when set, outcome_copy, and `status` is not read
    const int *flags;
    int nflags;
    int *outcome, *outcome_copy;
    int rows, cols, tokens, ksplit;
    float out_scale;
};
int fp4_mfma_splits(int rows, int cols, int tokens);
int fp4_mfma_launch(const Fp4MfmaLaunch &launch, hipStream_t stream);

// ---------------------------------------------------------------- bf16 and 8-bit affine matvecs

// y[t][r] = bf16 row r of `weights` times x[t], eight column chains per row folded in the reference's tree
// (src/kernels.c:139-174), plus bias[r] (or 0.0f).  All pointers are device pointers.
struct Bf16Launch {
    const uint16_t *weights;  // [rows][cols]
    const float *x;           // [tokens][x_stride]
    const float *bias;        // [rows] or null
    float *y;                 // [tokens][y_stride]
    int rows, cols, tokens;
    int x_stride, y_stride;
};
bool bf16_is_tileable(const Bf16Launch &launch);
int bf16_launch(const Bf16Launch &launch, hipStream_t stream);

// y[t][r] = sum over c, one left-to-right chain, of ((float)byte * scale + bias) * x[t][c] with the scale and bias
// of the 64-element group that holds flat element r * cols + c (src/kernels.c:343-370).
struct Q8Launch {
    const uint8_t *vals;      // [rows][cols] bytes
    const uint8_t *scales;    // bf16 per 64 flat elements
    const uint8_t *biases;    // bf16 per 64 flat elements, or null (0.0f)
    const float *x;           // [tokens][x_stride]
    float *y;                 // [tokens][y_stride]
    int rows, cols, tokens;
    int x_stride, y_stride;
};
int q8_launch(const Q8Launch &launch, hipStream_t stream);

// ---------------------------------------------------------------- fp32 cells of a decoder block

// Each launcher enqueues kernels that do nothing when *status != 0 and set it to -1 (publishing nothing) when an
// input or a result is not finite.  kind: 0 rms norm (weight optional), 1 router input, 2 residual post-norm.
int norm_cell_launch(int kind, const float *x, const float *weight, const float *residual, float *out, int n, float eps,
                     float root, int *status, hipStream_t stream);
// Opens a feed-forward block: *status is written (0 or -1), not only set.
int ffn_pre_launch(const float *residual, const float *w1, const float *w2, const float *router_scale, float *norm_a,
                   float *norm_b, float *router_in, int n, float eps, int *status, hipStream_t stream);
int combine_cell_launch(const float *residual, const float *dense, const float *routed, const float *wd, const float *wr,
                        const float *wf, float *sum_scratch, float *out, int n, float eps, float scalar, int *status,
                        const int *other_status, const float *expert_out, const float *weights, int topk,
                        hipStream_t stream);
int softcap_cell_launch(float *logits, size_t n, float cap, int *status, hipStream_t stream);
int merge_status_launch(int *status, const int *other, hipStream_t stream);

// ---------------------------------------------------------------- MoE

struct MoeGeometry {
    int hidden;               // d_model
    int routed;               // d_ff
    int n_experts;
    int topk;
};

// Device workspace of one decode layer-step; sized by moe_workspace_bytes.
struct MoeWorkspace {
    Q4Job *gate_up_jobs;      // 2*topk jobs
    Q4Job *down_jobs;         // topk jobs
    float *gate;              // [topk][routed]
    float *up;                // [topk][routed]
    float *act;               // [topk][routed]
    float *expert_out;        // [topk][hidden]
    int *status;              // 0 ok, -1 router rejected its input
    int *arrivals;            // one counter per 64 rows of the layer output (MoeFuse::arrivals)
};

size_t moe_workspace_bytes(const MoeGeometry &g);
void moe_workspace_carve(const MoeGeometry &g, void *base, MoeWorkspace *ws);

// sorted_by_id = 0: descending logit order (what the reference function returns);
// 1: ascending expert id (what its callers turn that into before running experts)
int router_topk_launch(const float *logits, const float *per_expert_scale, int n_experts, int topk,
                       int sorted_by_id, int *selected, float *weights, int *status, hipStream_t stream);

// out == nullptr leaves the ordered weighted reduction of expert_out to the caller
int moe_decode_step_launch(const MoeGeometry &g, const uint8_t *pool, size_t expert_stride,
                           const float *logits, const float *per_expert_scale, const float *x,
                           int *selected, float *weights, float *expert_out, float *out,
                           const MoeWorkspace &ws, float code_scale, hipStream_t stream);

// tolerance class (q4_dot.hip); -1 when the geometry is not served (more than 256 experts, widths the streaming
// kernel does not take)
int moe_decode_step_t_launch(const MoeGeometry &g, const uint8_t *pool, size_t expert_stride, const float *logits,
                             const float *per_expert_scale, const float *x, int *selected, float *weights,
                             float *expert_out, float *out, const MoeWorkspace &ws, hipStream_t stream);

int moe_activate_launch(const float *gate, const float *up, float *act, size_t n, hipStream_t stream);
int moe_reduce_launch(const float *expert_out, const float *weights, int topk, int hidden, float *out,
                      const int *status, hipStream_t stream);

// Grouped prefill MoE (reference src/moe_group.c): rows bucketed per expert in
// ascending expert / token / rank order, gate-up and down on the MFMA kernel,
// ordered weighted reduction.  Device workspace sized by moe_prefill_workspace_bytes.
size_t moe_prefill_workspace_bytes(const MoeGeometry &g, int tokens);
// status_dev receives 0, or -1 for an invalid selection (then outputs are not written).
int moe_prefill_launch(const MoeGeometry &g, const uint8_t *pool, size_t expert_stride, int tokens,
                       const int *selected, const float *weights, const float *inputs, float *outputs,
                       int *group_rows, int *row_pairs, int *status_dev, void *workspace, hipStream_t stream);

// Zero `words` 32-bit words at dst with a kernel on `stream` (safe under graph capture, unlike a memset node).
int clear_words_launch(void *dst, size_t words, hipStream_t stream);
// Copy `words` 32-bit words with a kernel; src may be mapped pinned host memory (its device view).
int copy_words_launch(void *dst, const void *src, size_t words, hipStream_t stream);

// ---------------------------------------------------------------- formats (formats.hip)

int q4_decode_launch(const uint8_t *vals, const uint8_t *scales, const uint8_t *biases, size_t n, float *out,
                     hipStream_t stream);
int nvfp4_dequant_launch(const uint8_t *packed, const uint8_t *scales, float weight_global_scale, int R, int C, float *out,
                         hipStream_t stream);
int router_fixture_launch(int n_experts, int topk, uint64_t state, int layer, double locality, int *idx, float *w,
                          hipStream_t stream);

// ---------------------------------------------------------------- probes

// Decodes all 256 byte values through the fp8 and fp4 converters (device
// arrays of 256 and 512 floats).
int probe_converters_launch(float *fp8_values, float *fp4_values, hipStream_t stream);

}  // namespace mi355
