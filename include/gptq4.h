/*
 * gptq4.h - C ABI of the MI355X (gfx950) 4-bit GPTQ inference kernels.
 *
 * The reference (fpgaminer/GPTQ-triton) has no FFI: its hot path is two Triton JIT
 * kernels launched from Python.  Each entry point below replaces one such launch
 * site; the citation names it (paths relative to the reference checkout).
 *
 * Conventions
 *  - Every pointer is a DEVICE pointer owned by the caller.  The library never
 *    allocates or frees memory and never synchronises the device or the stream.
 *  - Work is enqueued on `stream` (a hipStream_t passed as void*; NULL = default
 *    stream).  Calls are stream-ordered and may be issued back to back.
 *  - Return value: 0 on success; a negative GPTQ4_E_* code when an argument is
 *    rejected on the host (nothing was launched); a positive value is a hipError_t
 *    reported by the launch.  Nothing throws, nothing exits.
 *  - Tensor layouts are the reference checkpoint layouts, row-major contiguous:
 *      qweight int32 [K/8, N]  bits [4t,4t+4) of word (r,n) = nibble of row k=8r+t
 *      qzeros  int32 [G, N/8]  bits [4t,4t+4) of word (g,c) = stored zero of col 8c+t
 *      scales  fp16  [G, N]
 *    with G = K / groupsize (groupsize == K, or -1, means one group).  A weight
 *    decodes as  w = fp16( float(q - (z + 1)) * float(s) )  - exactly one rounding.
 *  - `groupsize` must be -1, K, or a multiple of 128 that divides K; K % 128 == 0;
 *    N % 256 == 0 (what the reference accepts: quant_linear.py:244-257).
 *  - `perm` (nullable) is the act-order row permutation made by
 *    gptq4_actorder_sort_rows(): logical weight row j multiplies x[:, perm[j]] and
 *    belongs to group j / groupsize.  The calls gather the rows of x into the workspace
 *    with one small launch of their own and multiply from there (up to 1 GiB of rows; beyond
 *    that, or with more than 16 rows and a workspace without room for them, the tiled kernel
 *    gathers by itself, which is slower).
 *  - `workspace` holds split-K partial sums, arrival counters and, for a call with
 *    `perm`, the gathered activations (M * K * 2 bytes).  Size it with
 *    gptq4_workspace_bytes() (selector | GPTQ4_OP_WITH_PERM for such calls); its first GPTQ4_WS_HEAD_BYTES bytes
 *    (the arrival counters, then the region where the decode GEMV exchanges marked partial sums) must be zero
 *    before the FIRST call that uses it (each call leaves them zero again).  Word GPTQ4_WS_ERROR_WORD (32-bit
 *    words from the start) is the exception: a kernel whose bounded wait for another wave's partial sums ran
 *    out sets it to 1 and it stays set - the results of that call are not valid and the workspace has to be
 *    zeroed again before it is reused.  One workspace may be shared by all calls on one stream; calls that
 *    run concurrently on different streams need a workspace each.
 */
#ifndef GPTQ4_H
#define GPTQ4_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define GPTQ4_ABI_VERSION 2

/* host-side argument errors (returned negated: -GPTQ4_E_SHAPE ...) */
#define GPTQ4_E_NULL 1       /* a required pointer is NULL                       */
#define GPTQ4_E_SHAPE 2      /* K, N, M, B, S, H or D outside what is supported  */
#define GPTQ4_E_GROUPSIZE 3  /* groupsize does not divide K / not a multiple of 128 */
#define GPTQ4_E_WORKSPACE 4  /* workspace NULL or smaller than required          */
#define GPTQ4_E_ALIGN 5      /* a pointer is not 16-byte aligned                 */
#define GPTQ4_E_STATIC_LIMIT 6 /* gptq4_matmul_static: the call needs more scratch than the library holds */

/* head of a workspace, kept zero between calls: arrival counters, then marked partial sums (8 bytes each) */
#define GPTQ4_WS_COUNTER_BYTES 524288
#define GPTQ4_WS_TAGGED_BYTES (16u << 20)
#define GPTQ4_WS_HEAD_BYTES (GPTQ4_WS_COUNTER_BYTES + GPTQ4_WS_TAGGED_BYTES)
#define GPTQ4_WS_ERROR_WORD 1
#define GPTQ4_KV_AT_POSITION (-1)
/* scratch memory inside the library for gptq4_matmul_static: the head plus 8 MiB of partial sums */
#define GPTQ4_STATIC_SCRATCH_BYTES (GPTQ4_WS_HEAD_BYTES + (8u << 20))

/* operation selector for gptq4_workspace_bytes */
#define GPTQ4_OP_MATMUL 0
#define GPTQ4_OP_MLP_GATEUP 1
#define GPTQ4_OP_QKV_ROTARY 2
#define GPTQ4_OP_DECODE_ATTENTION 3 /* M = B * H, K = kv_capacity, N unused */
#define GPTQ4_OP_WITH_PERM 0x100    /* or-ed to a matmul selector: the call will pass `perm` */

int gptq4_abi_version(void);
const char *gptq4_strerror(int code);

/* Bytes of workspace an operation needs for M rows and N output columns
 * (N = I for MLP_GATEUP, N = 3*H*D for QKV_ROTARY; or GPTQ4_OP_WITH_PERM to the selector for
 * calls that pass `perm`: room for the gathered rows).  No reference counterpart: the
 * Triton kernels own a whole K loop per output tile; split-K across workgroups is
 * what fills 256 CUs on GEMV-sized problems. */
size_t gptq4_workspace_bytes(int op, int M, int K, int N);

/* W_out fp16 [K, N] = dequantised weight, bit-exact to the formula above.
 * Replaces the in-kernel decode of matmul4_kernel (quant_linear.py:177-188,211-212)
 * as a stand-alone materialisation; g_idx (nullable) is int32 [K], the group of each
 * row in the ORIGINAL checkpoint row order (quantize.py:253 is the default). */
int gptq4_dequant(const int32_t *qweight, const int32_t *qzeros, const void *scales,
                  const int32_t *g_idx, void *W_out, int K, int N, int groupsize,
                  void *stream);

/* Load-time act-order re-layout: qweight_out row j = qweight row perm[j] (nibble rows,
 * K of them).  With perm = stable argsort(g_idx) the rows of each group become
 * contiguous so the matmul kernels can index groups as j / groupsize.  The reference
 * has no act-order kernel path (quantize.py:41-42 rejects act-order with groups). */
int gptq4_actorder_sort_rows(const int32_t *qweight, const int32_t *perm,
                             int32_t *qweight_out, int K, int N, void *stream);

/* y fp16 [M, N] = x fp16 [M, K] @ dequant(qweight, qzeros, scales) (+ bias fp16 [N]).
 * fp16 operands, fp32 accumulation, one rounding to fp16, then an fp16 bias add.
 * Replaces triton_matmul4 / matmul4_kernel (quant_linear.py:125-283). */
int gptq4_matmul(const void *x, const int32_t *qweight, const int32_t *qzeros,
                 const void *scales, const int32_t *perm, const void *bias, void *y,
                 int M, int K, int N, int groupsize, void *workspace,
                 size_t workspace_bytes, void *stream);

/* gptq4_matmul for callers that cannot allocate device memory (code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc): no workspace argument - the workspace head (arrival counters, marked
 * partial sums) and 8 MiB of split-K partial sums live in a fixed array inside the library
 * (GPTQ4_STATIC_SCRATCH_BYTES = 24.5 MiB per GPU, held until the process ends), and the call itself allocates and
 * frees nothing.  No reference counterpart.
 * Same kernels and results as gptq4_matmul without `perm` (act-order calls need room for the gathered
 * rows: use gptq4_matmul).  Calls whose workspace requirement - gptq4_workspace_bytes(GPTQ4_OP_MATMUL, M, K, N) -
 * exceeds the array return -GPTQ4_E_STATIC_LIMIT and launch nothing; decode-sized calls fit up to
 * M * N <= 131072 (16 rows of 8192 columns, 8 of 16384).  Every call on one GPU shares that GPU's array:
 * calls that overlap in time on one GPU (different streams or threads) race; calls on one stream do not.
 * The first call on a device looks the array's address up (hipGetSymbolAddress); make that call outside
 * stream capture. */
int gptq4_matmul_static(const void *x, const int32_t *qweight, const int32_t *qzeros,
                        const void *scales, const void *bias, void *y, int M, int K, int N,
                        int groupsize, void *stream);

/* h fp16 [M, I] = silu(x @ Wgate) * (x @ Wup); SiLU and the product are taken on the
 * fp32 accumulators, one rounding to fp16.
 * Replaces triton_llama_mlp_4 / llama_mlp_fused_4_kernel (fused_mlp.py:109-302). */
int gptq4_mlp_gateup(const void *x, const int32_t *gate_qweight, const int32_t *gate_qzeros,
                     const void *gate_scales, const int32_t *up_qweight,
                     const int32_t *up_qzeros, const void *up_scales, const int32_t *perm,
                     void *h, int M, int K, int I, int groupsize, void *workspace,
                     size_t workspace_bytes, void *stream);

/* cos, sin float32 [max_pos, D/2]:  angle = float(p) * (1 / base^(2i/D)).
 * Stands in for the rotary_emb module the reference receives from its model
 * (fused_attention.py:98-101). */
int gptq4_rope_table(float *cos_out, float *sin_out, int max_pos, int D, float base,
                     void *stream);

/* Fused QKV projection + rotary embedding.  x fp16 [B*S, K]; packed weights have
 * N = 3*H*D columns in the order q, k, v.  position_ids int32 [B*S] index the
 * cos/sin tables ([max_pos, D/2] float32).  Outputs (fp16):
 *   q [B, H, S, D]                      rotated
 *   k [B, H, kv_capacity, D] rows kv_offset + s, rotated
 *   v [B, H, kv_capacity, D] rows kv_offset + s, as projected
 * kv_capacity = S and kv_offset = 0 give the reference's three [B,H,S,D] tensors;
 * other values write straight into a preallocated KV cache.  kv_offset =
 * GPTQ4_KV_AT_POSITION writes token (b, s) to cache row position_ids[b*S + s] (clamped
 * into [0, kv_capacity)): no argument changes from one decode step to the next, so a
 * captured HIP graph of the step can be replayed.
 * Replaces qkv_proj + split + view/transpose + apply_rotary_pos_emb
 * (fused_attention.py:91-102).  D must be 128. */
int gptq4_qkv_rotary(const void *x, const int32_t *qweight, const int32_t *qzeros,
                     const void *scales, const int32_t *perm, const int32_t *position_ids,
                     const float *cos_table, const float *sin_table, int max_pos,
                     void *q, void *k, void *v, int B, int S, int H, int D, int K,
                     int groupsize, int kv_capacity, int kv_offset, void *workspace,
                     size_t workspace_bytes, void *stream);

/* The two projections that read a normalised residual stream, with that residual add + RMSNorm
 * done by the matmul kernel itself (one launch less per decoder block and decode step):
 *   s = delta ? fp16(x + delta) : x;   if delta: sum_out = s;   xn = norm_weight * fp16(s * rsqrt(mean(s^2) + eps));
 * then gptq4_qkv_rotary / gptq4_mlp_gateup on xn.  x, delta (nullable), sum_out fp16 [M, K], norm_weight
 * fp16 [K]; bit-identical to gptq4_add_rmsnorm (or gptq4_rmsnorm) followed by the plain entry point.
 * Decode-sized calls only: M <= 4, K <= 8192 (else -GPTQ4_E_SHAPE: run the two calls); perm as in the
 * plain entry points.  Every workgroup normalises every row, so it is the faster way for one row (1.3-1.4 us
 * on top of the plain projection against a 4.7 us norm launch), about even for two, slower beyond.  sum_out must not be x or delta: other workgroups of the launch still read them.
 * No reference counterpart (the reference runs LlamaRMSNorm as separate torch kernels,
 * src/gptq_triton/__init__.py:32-47). */
int gptq4_norm_qkv_rotary(const void *x, const void *delta, const void *norm_weight, float eps, void *sum_out,
                          const int32_t *qweight, const int32_t *qzeros, const void *scales,
                          const int32_t *perm, const int32_t *position_ids, const float *cos_table,
                          const float *sin_table, int max_pos, void *q, void *k, void *v, int B, int S, int H, int D, int K,
                          int groupsize, int kv_capacity, int kv_offset, void *workspace,
                          size_t workspace_bytes, void *stream);
int gptq4_norm_mlp_gateup(const void *x, const void *delta, const void *norm_weight, float eps, void *sum_out,
                          const int32_t *gate_qweight, const int32_t *gate_qzeros, const void *gate_scales,
                          const int32_t *up_qweight, const int32_t *up_qzeros, const void *up_scales,
                          const int32_t *perm, void *h, int M, int K, int I, int groupsize, void *workspace,
                          size_t workspace_bytes, void *stream);

/* RMSNorm over the last dimension: y = weight * fp16(x * rsqrt(mean(x^2) + eps)), x and y
 * fp16 [M, H], weight fp16 [H], H a multiple of 8; statistics in fp32.  Stands in for the
 * LlamaRMSNorm modules of the model the reference builds and runs between its fused blocks
 * (src/gptq_triton/__init__.py:32-47; the quantised linears are the only modules it swaps).
 * y_index (nullable) int32 [H], a permutation of 0..H-1: value f of a row is then stored at
 * y[m, y_index[f]] (y must not alias an input) - with the inverse of an act-order projection's
 * `perm`, y comes out in the order of that projection's sorted rows and the projection is called
 * without `perm`. */
int gptq4_rmsnorm(const void *x, const void *weight, void *y, const int32_t *y_index, int M, int H,
                  float eps, void *stream);

/* The residual add that precedes every RMSNorm of a decoder layer, fused with it:
 * sum_out = fp16(x + delta) (may alias x), y = RMSNorm(sum_out).  Same shapes and y_index as
 * above.  In the reference these are two torch ops of the HF decoder layer around its patched
 * blocks. */
int gptq4_add_rmsnorm(const void *x, const void *delta, const void *weight, void *sum_out, void *y,
                      const int32_t *y_index, int M, int H, float eps, void *stream);

/* Attention of ONE query token per sequence over a preallocated KV cache: for each (b, h)
 * softmax(q . K[0..positions[b]]^T * scale) . V[0..positions[b]], in fp32, written as fp16
 * out [B, H*D] (the layout o_proj consumes).  q fp16 [B, H, 1, D]; k_cache, v_cache fp16
 * [B, H, kv_capacity, D]; positions int32 [B] (clamped into [0, kv_capacity)); D must be
 * 128; B * H <= 4096.  out_index (nullable) int32 [H*D], a permutation of 0..H*D-1: feature f of
 * a row is then stored at out[b, out_index[f]] - with the inverse of an act-order o_proj's `perm`
 * the context comes out in the order of that projection's sorted rows, and o_proj is called
 * without `perm`.  workspace as for the matmuls (zeroed head, gptq4_workspace_bytes with
 * GPTQ4_OP_DECODE_ATTENTION).  Replaces the attention core of QuantLlamaAttention.forward for q_len == 1
 * (fused_attention.py:118-148: scores, mask, fp32 softmax, weighted sum, transpose). */
int gptq4_decode_attention(const void *q, const void *k_cache, const void *v_cache,
                           const int32_t *positions, void *out, const int32_t *out_index,
                           int B, int H, int D,
                           int kv_capacity, float scale, void *workspace,
                           size_t workspace_bytes, void *stream);

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
 * fit), a reserved value, polls before a wait gives up (0 = default, about seconds), and a workgroup that never
 * stores its partial sums (-1 = none; lets a test see the bounded waits give up with every kernel exiting normally). */
void gptq4_set_chain_tuning(int ring_slots, int reserved, unsigned spin_limit, int skip_flag_wg);

/* Host-side launch tuning of the small-M kernels, for measurements: words per lane and
 * load (1, 2 or 4: strips of 16, 32 or 64 columns), batches of loads in flight per
 * wave (1..4) and the split-K factor; 0 = automatic for each.  words + 10 (10 = automatic width): the workgroups
 * that share a tile always exchange plain partial sums under an arrival counter; words + 20: marked 8-byte values
 * wherever those fit GPTQ4_WS_TAGGED_BYTES (by default: up to 4 rows and few splits).  Process-wide; not
 * thread-safe against concurrent launches.  No reference counterpart (the reference
 * tunes through Triton's autotuner, custom_autotune.py:12-172). */
void gptq4_set_tuning(int words, int depth, int splitk);

/* Same for the tiled (M > 16) kernel: workgroup tile (mt = 2: 128 x 128, mt = 4: 128 x 256
 * outputs; half as wide for the fused gate/up) and the split-K factor; 0 = automatic.
 * mt = 10, 12 or 14: the same tile choice, and act-order calls use the tiled kernel's own
 * gather of the activations instead of the copy staged in the workspace.  mt = 200: the streamed
 * schedule (K tiles of all wide tiles dealt evenly to the resident workgroups; never chosen
 * automatically, it measured slower) wherever it can run, mt = 100: never; mt = 300: never cut a call into two
 * launches over adjacent column ranges, mt = 400: never cut the column panels past the last whole round of wide tiles
 * along K inside the launch (the mid-M kernel's launches included), mt = 500: neither (both are done automatically where the wide-tile count is just above
 * a multiple of the CU count); tile and split automatic with all five. */
void gptq4_set_gemm_tuning(int mt, int splitk);

/* Same for the mid-M kernel (M > 16 with too few wide tiles for the tiled kernel; K is split
 * across the four or eight waves of a workgroup): mode 0 = never use it, 1 = where it is the faster
 * kernel, 2 = wherever it can run; 32-row blocks per row tile (1, 2; 10 + that, or 10 alone, also
 * selects 128-column strips for plain projections, a plain 1 or 2 the 64-column strips; 100 + any of
 * these: four waves per workgroup, 200 +: eight where they fit; 1000 + any of these: the rotary epilogue on tiles
 * of 32 columns of a head plus their 32 rotation partners instead of whole heads, 2000 +: never) and the split-K
 * factor across workgroups; 0 = automatic. */
void gptq4_set_midm_tuning(int mode, int mt, int splitk);

/* Same for the balanced decode GEMV (M <= 4): mode 0 = never use it, 1 = where it is the
 * faster kernel (one row, SiLU*mul epilogue), 2 = wherever it can run; units in
 * flight per wave (1..3), waves per workgroup (4, 8, 16), waves per CU (4..32), 0 =
 * automatic. */
void gptq4_set_gemv_tuning(int mode, int depth, int waves, int waves_per_cu);
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

#ifdef __cplusplus
}
#endif
#endif /* GPTQ4_H */
