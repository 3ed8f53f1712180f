// Host-side contracts between the C ABI (gptq4_api.hip) and the kernel launchers.
#pragma once

#include "gptq4_common.h"

// Kernel arguments are fetched with scalar loads where the compiler first needs them, and an early exit or a loop
// between two uses turns that into two or three dependent round trips to memory at the very start of a launch
// (0.5 - 0.7 us each, with nothing else in flight).  Naming the arguments of the streaming loop and of the exchange
// in one empty asm statement at the top of a kernel makes the compiler fetch them together.
#define GPTQ4_FETCH_MATMUL_ARGS(p)                                                                                        \
    asm volatile("" ::"s"((p).x), "s"((p).w[0].qweight), "s"((p).w[0].qzeros), "s"((p).w[0].scales), "s"((p).w[1].qweight), \
                 "s"((p).w[1].qzeros), "s"((p).w[1].scales), "s"((p).partials), "s"((p).counters), "s"((p).tagged), "s"((p).y), \
                 "s"((p).M), "s"((p).K), "s"((p).N), "s"((p).groupsize), "s"((p).splitk), "s"((p).tiles), "s"((p).slot_q),   \
                 "s"((p).slot_rem), "s"((p).batches_per_group))

// One quantised projection as the kernels see it.
struct QMat {
    const uint32_t *qweight;  // [K/8, N]
    const uint32_t *qzeros;   // [G, N/8]
    const half_t *scales;     // [G, N]
};

struct MatmulArgs {
    const half_t *x;  // [M, K]
    QMat w[2];        // w[1] only for EPI_SILU_MUL (w[0] = gate, w[1] = up)
    float *partials;
    int *counters;
    uint64_t *tagged;     // small-M kernels: marked partial sums, GPTQ4_WS_TAGGED_BYTES of them behind the counters (split-K kernel: null = exchange through counters)
    uint32_t spin_limit;  // small-M kernels: polls of a slot before a finishing wave gives up
    half_t *y;  // [M, N] (EPI_PLAIN, EPI_SILU_MUL)
    const half_t *bias;
    const int32_t *perm;
    int M, K, N;
    // M > 16 kernels: the launch computes output columns [n_begin, n_begin + n_count) only (N stays the row length of
    // the weights and of the result); the whole matrix: 0, N
    int n_begin, n_count;
    int tail_first, tail_split;  // tiled kernel, wide unsplit tiles: see GemmPlan
    int groupsize;  // normalised: K when the caller passed -1
    int splitk;
    int tiles;
    int stream_b;  // tiled kernel: the packed words are in streaming order and w[].qzeros holds the {scale, zero} words (w[].scales unused)
    // small-M kernel: K batches (128 k each) dealt to splitk * 4 wave slots - slot i
    // gets slot_q batches, the first slot_rem slots one more.  Tiled kernel: K tiles
    // (64 k each) dealt to splitk splits the same way.
    int slot_q, slot_rem;
    int batches_per_group;  // groupsize / 128
    int groups;             // K / groupsize
    // balanced GEMV: units = tiles * nb are dealt to waves, slot_q each and one more for
    // the first slot_rem.  Divisions run through host-made reciprocals floor(2^32 / d) + 1:
    // of batches_per_group (batch -> group), nb, slot_q and slot_q + 1.  The x slice of a
    // wave has 1 << m_shift >= M rows per unit.
    uint32_t group_magic;
    int m_shift;
    int nb;
    uint32_t nb_magic, q_magic, q1_magic;
    int lds_wave_chunks;  // 16-byte chunks of LDS per wave
    int x_chunks_max;     // chunks of the largest x slice: (slot_q + 1) << (4 + m_shift)
    int max_contrib;      // partial-sum slots per tile
    RopeArgs rope;          // EPI_ROPE only
    // fused residual add + RMSNorm of the input (small-M kernels): when nrm_weight is set, x is the
    // residual stream and the kernel multiplies with nrm_weight * rmsnorm(x (+ nrm_delta)); the sums
    // x + nrm_delta go to nrm_sum_out (not aliasing x or nrm_delta: other workgroups still read them)
    const half_t *nrm_delta;
    const half_t *nrm_weight;
    half_t *nrm_sum_out;
    float nrm_eps;
};

// Launch shape of the small-M kernel.
struct SkinnyPlan {
    int words;   // packed words per lane and load: strip width = 16 * words columns
    int depth;   // batches of loads kept in flight per wave
    int splitk;  // workgroups sharing one tile
    int waves;   // waves per workgroup (4, 8 or 16), each with its own K range
    int tiles;
};
struct SkinnyTuning {
    int words, depth, splitk, waves;  // 0 = automatic
    int exchange;                     // 0 = automatic, 1 = always arrival counters and plain partial sums
};
extern SkinnyTuning g_skinny_tuning;
// standard_shape: ignore the tuning overrides of words, depth and waves (the split is still tunable)
SkinnyPlan skinny_plan(int epi, int M, int N, int K, bool standard_shape = false);
// Small-M (M <= 16) split-K matrix-core GEMV.  Returns hipError_t.
int launch_skinny(int epi, const MatmulArgs &a, const SkinnyPlan &plan, hipStream_t stream);
// Balanced decode GEMV (M <= GEMV_MAX_M): (tile, batch) units dealt evenly to waves.
struct GemvPlan {
    int depth, waves;         // units in flight per wave, waves per workgroup
    int tiles, nb;            // column tiles, 128-k batches per tile
    int workgroups;
    int q, r;                 // units per wave, waves with one more
    int m_shift, lds_wave_chunks, max_contrib;
    size_t lds_bytes;
    bool ok;                  // false: use another kernel
};
struct GemvTuning {
    int mode;                        // 0 never, 1 where it is the faster kernel, 2 wherever it can run
    int depth, waves, waves_per_cu;  // 0 = automatic
    uint32_t spin_limit;             // 0 = the default bound on a finishing wave's polls
};
extern GemvTuning g_gemv_tuning;
// norm: plan for the variant that normalises its own input (automatic launch shape, room for the rows in LDS)
GemvPlan gemv_plan(int epi, int M, int N, int K, bool norm = false);
// bytes of marked partial sums (8 per value) the plan exchanges; a plan is only ok while they fit GPTQ4_WS_TAGGED_BYTES
size_t gemv_tagged_bytes(const GemvPlan &plan, int M, int epi);
int launch_gemv(int epi, MatmulArgs &a, const GemvPlan &plan, hipStream_t stream);
// Launch shape of the tiled kernel.
struct GemmPlan {
    int mt;      // 32-row tiles per wave: 2 = 128 x 128 workgroup tile (2 x 2 waves), 4 = 128 x 256 (1 x 4 waves)
    int splitk;  // workgroups sharing one tile along K
    int tiles;
    double score;  // expected efficiency of the choice: fill of the chip / cost of the splits (1 where the tile count is large)
    int streamed;  // 0, or the grid of the streamed schedule (wide tiles, K tiles of all tiles dealt evenly to that many workgroups)
    // wide tiles, unsplit: tiles [0, tail_first) whole, the tiles from tail_first on cut into tail_split parts along K
    // (1 = no tile is cut)
    int tail_first, tail_split;
};
struct GemmTuning {
    int mt, splitk;  // 0 = automatic
    int own_gather;  // 1: act-order calls run the tiled kernel's own gather instead of staging the activations
    int streamed;    // 0 = automatic, 1 = never, 2 = wherever it can run
    int parts;       // 0 = automatic, 1 = never cut a call into two launches over column ranges
    int tail;        // 0 = automatic, 1 = never cut the tiles past a whole number of rounds along K
};
extern GemmTuning g_gemm_tuning;
// has_perm: the kernel will gather act-order activations itself (no streamed schedule then); allow_streamed = false:
// the call must not plan the streamed schedule (its partial sums would not fit the caller's scratch memory)
GemmPlan gemm_plan(int epi, int M, int N, int K, bool has_perm = false, bool allow_streamed = true);
size_t gemm_partial_bytes(const GemmPlan &plan);
// Tiled matrix-core GEMM for any M.  Returns hipError_t.
int launch_gemm(int epi, const MatmulArgs &a, const GemmPlan &plan, hipStream_t stream);

// Launch shape of the mid-M kernel (K split across the waves of a workgroup).
struct KslicePlan {
    int mt;      // 32-row blocks per row tile (1 or 2)
    int splitk;  // workgroups sharing one tile along K, on top of the split inside the workgroup
    int tiles;
    bool wide;   // plain epilogue: 128-column strips (two blocks per wave tile) instead of 64
    int waves;   // waves per workgroup, each with its own slice of K (4 or 8)
    bool paired; // rotary epilogue: tiles of 32 columns of a head plus their 32 rotation partners instead of whole heads
    bool ok;     // false: the shape needs another kernel
    // tail_split > 1 (only with splitk == 1): tiles [0, tail_first) whole, every later one - the last column strips
    // of the launch, all their row tiles - shared by tail_split workgroups along K
    int tail_first, tail_split;
};
struct KsliceTuning {
    int mode;        // 0 never, 1 where it is the faster kernel, 2 wherever it can run
    int mt, splitk;  // 0 = automatic
    int wide;        // plain epilogue: 1 = 128-column strips, -1 = 64-column strips, 0 = automatic
    int waves;       // waves per workgroup: 4, 8, 0 = automatic
    int paired;      // rotary epilogue, tiles of 32 + 32 paired columns: 0 = automatic, 1 = always, 2 = never
};
extern KsliceTuning g_kslice_tuning;
KslicePlan kslice_plan(int epi, int M, int N, int K, bool has_perm);
size_t kslice_partial_bytes(int epi, const KslicePlan &plan);
int launch_kslice(int epi, const MatmulArgs &a, const KslicePlan &plan, hipStream_t stream);

// ---- Streaming-order layout (gptq4_stream.hip) ------------------------------------------------------------------
// One quantised projection in streaming order: per strip of 16 output columns and per unit of 128 input rows one
// contiguous 1 KiB block; lane l = 16 * r + c of a wave (r = 0..3, c = 0..15) owns bytes [16 * l, 16 * l + 16) of
// the block: the packed words of the 8-row blocks 4 * r + j (j = 0..3) of the unit, column c of the strip - the B
// operands of four v_mfma_f32_16x16x32_f16 steps.  Blocks are ordered [strip][unit].  `meta` holds one word per
// (strip, group, column): fp16 scale bits | stored zero << 16, ordered [strip][group][column].
struct SMat {
    const uint32_t *w;
    const uint32_t *meta;
};

struct StreamArgs {
    // (what a wave needs before its first load comes first)
    const half_t *x;  // [M, K]
    SMat m[2];        // m[1]: the up projection (EPI_SILU_MUL) or m[0] again (EPI_ROPE: the rotation partners' strips)
    int M, K, N;
    int nb;      // units per strip: K / 128
    int groups;  // K / groupsize
    int batches_per_group;
    uint32_t group_magic;
    int q, r;  // units per workgroup, and how many workgroups take one more
    uint32_t nb_magic;
    int xrow;     // 16-byte chunks per row of the activations in LDS
    int red_off;  // 16-byte chunks of LDS in front of the partial-sum slots
    int m_magic;  // ceil(2^16 / M)
    uint64_t *tagged;  // marked partial sums, one slot per workgroup
    uint32_t q_magic, q1_magic;
    int nat_off;  // NORM: 16-byte chunks of LDS in front of the normalised rows in natural order
    uint32_t spin_limit;
    int *counters;     // the workspace's counter region (error word)
    half_t *y;
    const half_t *bias;
    const int32_t *perm;
    RopeArgs rope;
    const half_t *nrm_delta;
    const half_t *nrm_weight;
    half_t *nrm_sum_out;
    float nrm_eps;
};

struct StreamPlan {
    int waves, depth;  // waves per workgroup (8 or 16), units in flight per wave
    int workgroups;
    int tiles, nb;
    int strips;  // tiles per unit (2 in the kernel for 5 .. 16 rows where the tile count is even)
    int q, r;
    int pieces;  // most tiles a workgroup's range touches
    int xrow, red_off, nat_off;
    size_t lds_bytes;
    bool ok;
    bool tall;  // 5 .. 16 rows: the kernel that fetches its A operand with every unit
};
struct StreamTuning {
    int waves, depth;  // 0 = automatic
};
extern StreamTuning g_stream_tuning;
enum { STREAM_MAX_M = 4, STREAM_TALL_MAX_M = 16 };  // rows with the activations in LDS (and the norm inside); rows at all
StreamPlan stream_plan(int epi, int M, int N, int K, bool norm);
int launch_stream(int epi, StreamArgs &a, const StreamPlan &plan, bool nomath, hipStream_t stream);
int launch_stream_pack(const uint32_t *qweight, const uint32_t *qzeros, const half_t *scales, uint32_t *sw, uint32_t *meta,
                       int K, int N, int groupsize, hipStream_t stream);
int launch_stream_unpack(const uint32_t *sw, const uint32_t *meta, uint32_t *qweight, uint32_t *qzeros, half_t *scales,
                         int K, int N, int groupsize, hipStream_t stream);
int launch_stream_dequant(const uint32_t *sw, const uint32_t *meta, half_t *out, int K, int N, int groupsize, hipStream_t stream);

int launch_dequant(const uint32_t *qweight, const uint32_t *qzeros, const half_t *scales,
                   const int32_t *g_idx, half_t *out, int K, int N, int groupsize,
                   hipStream_t stream);
int launch_sort_rows(const uint32_t *qweight, const int32_t *perm, uint32_t *out, int K, int N,
                     hipStream_t stream);
// out[m][j] = x[m][perm[j]] for M rows of K values.
int launch_gather_cols(const half_t *x, const int32_t *perm, half_t *out, int M, int K, hipStream_t stream);
int launch_rope_table(float *cos_out, float *sin_out, int max_pos, int D, float base,
                      hipStream_t stream);
// Decoder-side operators (gptq4_decoder.hip).
int launch_rmsnorm(const half_t *x, const half_t *delta, const half_t *w, half_t *sum_out, half_t *y, const int32_t *y_index,
                   int M, int H, float eps, hipStream_t stream);
size_t attn_decode_partial_bytes(int BH, int capacity);
size_t head_argmax_partial_bytes();
int launch_head_argmax(const half_t *x, const half_t *w, long long *out, float *part, int *counters, int B, int K, int V, hipStream_t stream);
int launch_attn_prefill(const half_t *q, const half_t *kc, const half_t *vc, half_t *out, int B, int H, int S, int capacity, int past,
                        float scale, hipStream_t stream);
int launch_attn_decode(const half_t *q, const half_t *kc, const half_t *vc, const int *positions, half_t *out,
                       const int32_t *out_index, int B, int H, int capacity, float scale, int *counters, float *partials, hipStream_t stream);

// Compute units and XCDs of the current device, asked once per device (hipDeviceProp_t / hipDeviceAttributeNumberOfXccs).
// Launch plans size their grids from it.  Where no device can be asked (plans made on a machine without a GPU, e.g.
// gptq4_workspace_bytes in a host-only test) it answers with MI355X's 256 CUs in 8 XCDs.
struct DeviceShape {
    int cus, xcds;
};
DeviceShape device_shape();

// arrival counters sit one per 128-byte line: atomics on one line are served one after
// the other by the memory side
enum { COUNTER_STRIDE = 32 };
// word of the counter region (between two counter lines' first words) that a kernel sets when a bounded wait ran out
enum { EXCHANGE_ERROR_WORD = 1 };
// act-order: activations up to this many bytes are gathered into the workspace ahead of the kernel
constexpr size_t ACT_ORDER_STAGE_MAX = (size_t)1 << 30;
enum { GEMV_MAX_M = 4, SKINNY_MAX_M = 16, SKINNY_MAX_SPLITK = 16, SKINNY_MAX_TILES = 4096, GEMM_MAX_SPLITK = 16 };
