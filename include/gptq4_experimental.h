/*
 * gptq4_experimental.h - entry points of libgptq4.so that are NOT part of the stable boundary (include/gptq4.h):
 * launch-tuning and test hooks of the kernels, a diagnostic, and a measured-and-slower design kept for its tests.
 * Nothing here is needed to use the library; signatures may change without a change of GPTQ4_ABI_VERSION.  All
 * setters are process-wide and not thread-safe against concurrent launches.  No reference counterpart (the
 * reference tunes through Triton's autotuner, custom_autotune.py:12-172).
 */
#ifndef GPTQ4_EXPERIMENTAL_H
#define GPTQ4_EXPERIMENTAL_H

#include "gptq4.h"

#ifdef __cplusplus
extern "C" {
#endif

/* first argument of gptq4_set_tuning (split-K decode kernel): words per lane, optionally with an exchange choice added */
enum gptq4_skinny_words {
    GPTQ4_SKINNY_AUTO = 0,
    GPTQ4_SKINNY_WORDS_1 = 1, /* strips of 16 columns */
    GPTQ4_SKINNY_WORDS_2 = 2, /* 32 */
    GPTQ4_SKINNY_WORDS_4 = 4, /* 64 */
    GPTQ4_SKINNY_EXCHANGE_COUNTERS = 10, /* + words: partial sums always under an arrival counter */
    GPTQ4_SKINNY_EXCHANGE_MARKED = 20    /* + words: marked 8-byte values wherever they fit */
};
/* first argument of gptq4_set_gemm_tuning (tiled kernel) */
enum gptq4_gemm_tile {
    GPTQ4_GEMM_AUTO = 0,
    GPTQ4_GEMM_TILE_128x128 = 2,
    GPTQ4_GEMM_TILE_128x256 = 4,
    GPTQ4_GEMM_OWN_GATHER = 10,   /* + tile: act-order calls gather inside the tiled kernel */
    GPTQ4_GEMM_NO_STREAMED = 100, /* never the streamed schedule */
    GPTQ4_GEMM_STREAMED = 200,    /* the streamed schedule wherever it can run */
    GPTQ4_GEMM_NO_PARTS = 300,    /* never two launches over column ranges */
    GPTQ4_GEMM_NO_TAIL = 400,     /* never cut the last column panels along K */
    GPTQ4_GEMM_NO_PARTS_NO_TAIL = 500
};
/* second argument of gptq4_set_midm_tuning (mid-M kernel): a sum of one value per group */
enum gptq4_midm_shape {
    GPTQ4_MIDM_AUTO = 0,
    GPTQ4_MIDM_ROWS_32 = 1,
    GPTQ4_MIDM_ROWS_64 = 2,
    GPTQ4_MIDM_WIDE_STRIPS = 10, /* 128-column strips for plain projections */
    GPTQ4_MIDM_WAVES_4 = 100,
    GPTQ4_MIDM_WAVES_8 = 200,
    GPTQ4_MIDM_PAIRED = 1000,    /* rotary epilogue on 32 + 32 paired columns */
    GPTQ4_MIDM_NOT_PAIRED = 2000
};
enum gptq4_kernel_mode { GPTQ4_MODE_NEVER = 0, GPTQ4_MODE_WHERE_FASTER = 1, GPTQ4_MODE_WHEREVER_POSSIBLE = 2 };

/* ---- Chained decode launch: several decode-sized projections in ONE persistent launch ----------------------
 * A decode step is a chain of small projections, each streaming its weights once; launched one by one, about
 * 6 us of every 6-15 us launch are launch floor, prologue, first-load latency and partial-sum exchange, during
 * which HBM idles.  gptq4_decode_chain runs a list of up to 8 "phases" on one resident grid (one workgroup per
 * CU) that streams the weights of all phases as one sequence: the loads of the next phase are in flight while
 * the one before is handed over.  No reference counterpart: the reference launches one Triton kernel per
 * projection (quant_linear.py:264-274, fused_mlp.py:286-297) with the torch ops of the decoder layer between
 * them.
 *
 * A phase is a 4-bit projection (or a gate/up pair: up_* set) of M <= 4 rows.  `input` says what it multiplies:
 *   GPTQ4_IN_ROWS       x fp16 [M, K], in memory before the launch
 *   GPTQ4_IN_NORM_ROWS  norm_weight * rmsnorm(x (+ delta)), x and delta in memory before the launch; the sums
 *                       x + delta go to sum_out (nullable)
 *   GPTQ4_IN_PREV       the output of the phase before it: fp16(sums) (+ bias) of a projection,
 *                       fp16(silu(gate) * up) of a pair; its N is this phase's K
 *   GPTQ4_IN_NORM_PREV  norm_weight * rmsnorm(x + previous output): x fp16 [M, K] is the residual stream (in
 *                       memory before the launch, or the sum_out of an earlier phase); sums to sum_out (nullable)
 * (the rounding order of gptq4_add_rmsnorm / gptq4_matmul / gptq4_mlp_gateup run one after the other; only the
 * order in which fp32 partial sums are added differs, fixed for a given shape and GPU).  `output`:
 *   GPTQ4_OUT_NONE      only the next phase reads it (which must then be IN_PREV / IN_NORM_PREV)
 *   GPTQ4_OUT_ROWS      y fp16 [M, N] is written as well (a pair writes silu(gate) * up)
 *   GPTQ4_OUT_ROPE      N = 3 * H * 128 columns q, k, v: rotary + head-major stores as gptq4_qkv_rotary with one
 *                       token per sequence (B = M, S = 1); nothing can read it as IN_PREV
 * K % 128 == 0, N % 256 == 0, groupsize as elsewhere; norm inputs need K <= 8192; `perm` must be NULL (act-order
 * inputs are not taken).  sum_out must not be x or delta.
 *
 * Workspace: gptq4_chain_workspace_bytes() bytes, 256-byte aligned, ZERO before the first launch; it carries
 * state from launch to launch (do not clear it between launches, do not share it with the other entry points,
 * one per stream).  All waits inside the launch are bounded: if a workgroup ever gives up (the grid was not
 * resident as a whole, e.g. because another stream's kernel held CUs for seconds), every workgroup returns,
 * outputs are undefined and the int32 at byte offset 4 of the workspace is set to 1 - later launches on that
 * workspace then return at once until the caller clears it (hipMemsetAsync the whole workspace, outside a graph).
 * Launch nothing else on other streams that needs the whole GPU for long while a chain runs. */
#define GPTQ4_IN_ROWS 0
#define GPTQ4_IN_NORM_ROWS 1
#define GPTQ4_IN_PREV 2
#define GPTQ4_IN_NORM_PREV 3
#define GPTQ4_OUT_NONE 0
#define GPTQ4_OUT_ROWS 1
#define GPTQ4_OUT_ROPE 2
#define GPTQ4_CHAIN_MAX_PHASES 8
#define GPTQ4_CHAIN_MAX_M 4
#define GPTQ4_CHAIN_ERROR_OFFSET 4

typedef struct gptq4_phase {
    const int32_t *qweight, *qzeros;
    const void *scales;
    const int32_t *up_qweight, *up_qzeros; /* all three set: qweight.. is gate, this is up */
    const void *up_scales;
    const int32_t *perm; /* must be NULL */
    const void *x, *delta, *norm_weight;
    void *sum_out;
    void *y;
    const void *bias;
    /* GPTQ4_OUT_ROPE */
    const int32_t *position_ids; /* [M] */
    const float *cos_table, *sin_table;
    void *q, *k, *v;
    int K, N, groupsize;
    int input, output;
    float eps;
    int H, max_pos, kv_capacity, kv_offset;
} gptq4_phase_t;

/* 0 if the list is not one gptq4_decode_chain accepts */
size_t gptq4_chain_workspace_bytes(const gptq4_phase_t *phases, int nphases, int M);
int gptq4_decode_chain(const gptq4_phase_t *phases, int nphases, int M, void *workspace,
                       size_t workspace_bytes, void *stream);
/* Measurement and test knobs of the chained launch: units of LDS ring per streaming wave (2..4, 0 = as many as
 * fit), a reserved value, polls before a wait gives up (0 = default: 16384, tens of milliseconds), and a workgroup that never
 * stores its partial sums (-1 = none; lets a test see the bounded waits give up with every kernel exiting normally). */
void gptq4_set_chain_tuning(int ring_slots, int reserved, unsigned spin_limit, int skip_flag_wg);

/* Host-side launch tuning of the small-M kernels, for measurements: words per lane and
 * load (1, 2 or 4: strips of 16, 32 or 64 columns), batches of loads in flight per
 * wave (1..4) and the split-K factor; 0 = automatic for each.  words + 10 (10 = automatic width): the workgroups
 * that share a tile always exchange plain partial sums under an arrival counter; words + 20: marked 8-byte values
 * wherever those fit GPTQ4_WS_TAGGED_BYTES (by default: up to 4 rows and few splits).  Process-wide; not
 * thread-safe against concurrent launches.  No reference counterpart (the reference
 * tunes through Triton's autotuner, custom_autotune.py:12-172). */
void gptq4_set_tuning(int words /* enum gptq4_skinny_words */, int depth, int splitk);

/* Same for the tiled (M > 16) kernel: workgroup tile (mt = 2: 128 x 128, mt = 4: 128 x 256
 * outputs; half as wide for the fused gate/up) and the split-K factor; 0 = automatic.
 * mt = 10, 12 or 14: the same tile choice, and act-order calls use the tiled kernel's own
 * gather of the activations instead of the copy staged in the workspace.  mt = 200: the streamed
 * schedule (K tiles of all wide tiles dealt evenly to the resident workgroups; never chosen
 * automatically, it measured slower) wherever it can run, mt = 100: never; mt = 300: never cut a call into two
 * launches over adjacent column ranges, mt = 400: never cut the column panels past the last whole round of wide tiles
 * along K inside the launch (the mid-M kernel's launches included), mt = 500: neither (both are done automatically where the wide-tile count is just above
 * a multiple of the CU count); tile and split automatic with all five. */
void gptq4_set_gemm_tuning(int mt /* enum gptq4_gemm_tile */, int splitk);

/* Same for the mid-M kernel (M > 16 with too few wide tiles for the tiled kernel; K is split
 * across the four or eight waves of a workgroup): mode 0 = never use it, 1 = where it is the faster
 * kernel, 2 = wherever it can run; 32-row blocks per row tile (1, 2; 10 + that, or 10 alone, also
 * selects 128-column strips for plain projections, a plain 1 or 2 the 64-column strips; 100 + any of
 * these: four waves per workgroup, 200 +: eight where they fit; 1000 + any of these: the rotary epilogue on tiles
 * of 32 columns of a head plus their 32 rotation partners instead of whole heads, 2000 +: never) and the split-K
 * factor across workgroups; 0 = automatic. */
void gptq4_set_midm_tuning(int mode /* enum gptq4_kernel_mode */, int mt /* enum gptq4_midm_shape */, int splitk);

/* Same for the balanced decode GEMV (M <= 4): mode 0 = never use it, 1 = where it is the
 * faster kernel (one row, SiLU*mul epilogue), 2 = wherever it can run; units in
 * flight per wave (1..3), waves per workgroup (4, 8, 16), waves per CU (4..32), 0 =
 * automatic. */
void gptq4_set_gemv_tuning(int mode /* enum gptq4_kernel_mode */, int depth, int waves, int waves_per_cu);
/* How a call with more than 16 rows is launched: as one launch over all N output columns (returns 1) or as two
 * launches over adjacent column ranges (returns 2; begin[i], cols[i] describe them) - the second where the count of
 * wide tiles is just above a multiple of the CU count, so that a few left-over tiles do not cost a round of their
 * own.  `op` is a GPTQ4_OP_* selector (N of one matrix for the gate/up pair); begin and cols have room for two
 * values (or are NULL).  For diagnostics and tests; no reference counterpart. */
int gptq4_column_parts(int op, int M, int K, int N, int *begin, int *cols);

/* How often a finishing wave of the small-M kernels polls for another wave's marked partial sums before it gives up
 * and sets GPTQ4_WS_ERROR_WORD (0 = the default, about four million polls).  0xFFFFFFFF is the hook for tests of
 * that error path: every finishing wave polls once and gives up whatever it found, and every kernel still ends
 * normally.  No reference counterpart. */
void gptq4_set_exchange_spin_limit(unsigned polls);

/* Launch shape of the streaming-order decode kernel: waves per workgroup (8 or 16) and units of loads in flight per
 * wave (1..3); 0 = automatic.  depth + 10: the kernel for 5 .. 16 rows takes one tile per unit of loads everywhere, depth + 20: two wherever they can run. */
void gptq4_set_stream_tuning(int waves, int depth);

/* The streaming-order kernel's launch with the decode and the matrix-core instructions left out: the same loads,
 * waits, LDS traffic and stores, no arithmetic (outputs are meaningless).  For `bench.py --floor-probe`: what the
 * access pattern alone costs.  op = GPTQ4_OP_MATMUL (up_* NULL) or GPTQ4_OP_MLP_GATEUP. */
int gptq4_stream_probe(int op, const void *x, const int32_t *sweight, const int32_t *smeta,
                       const int32_t *up_sweight, const int32_t *up_smeta, void *y, int M, int K, int N,
                       int groupsize, void *workspace, size_t workspace_bytes, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* GPTQ4_EXPERIMENTAL_H */
