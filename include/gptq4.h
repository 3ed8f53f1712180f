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

#define GPTQ4_ABI_VERSION 3

/* host-side argument errors (returned negated: -GPTQ4_E_SHAPE ...) */
#define GPTQ4_E_NULL 1       /* a required pointer is NULL                       */
#define GPTQ4_E_SHAPE 2      /* K, N, M, B, S, H or D outside what is supported  */
#define GPTQ4_E_GROUPSIZE 3  /* groupsize does not divide K / not a multiple of 128 */
#define GPTQ4_E_WORKSPACE 4  /* workspace NULL or smaller than required          */
#define GPTQ4_E_ALIGN 5      /* a pointer is not 16-byte aligned                 */
#define GPTQ4_E_STATIC_LIMIT 6 /* gptq4_matmul_static: the call needs more scratch than the library holds */
#define GPTQ4_E_EXCHANGE 7   /* gptq4_static_status: a bounded wait between workgroups ran out (error word set) */

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
/* The library's array is private, so these two do for it what a caller does with its own workspace (no reference
 * counterpart either).  gptq4_static_status waits for `stream` and returns 0, or -GPTQ4_E_EXCHANGE when a
 * gptq4_matmul_static call on this GPU gave up its bounded wait (GPTQ4_WS_ERROR_WORD set: that call's result is
 * invalid, and late partial sums may spoil later calls until the head is zeroed).  gptq4_static_reset zeroes the
 * head of the array on `stream` (a memset node: not under stream capture).  Neither allocates.  After an error:
 * let the GPU drain (gptq4_static_status did), then gptq4_static_reset. */
int gptq4_static_status(void *stream);
int gptq4_static_reset(void *stream);

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

/* The end of a greedy decode step in one launch: out[b] = argmax over v of fp16(x[b] . weight[v]) - the fp16 lm_head
 * (weight fp16 [V, K], row-major as nn.Linear keeps it; no bias) and the argmax of its output, the lowest index among
 * equal logits.  x fp16 [B, K], B <= 16; out int64 [B]; K one of 4096, 5120, 6656, 8192 (else -GPTQ4_E_SHAPE: use a
 * dense GEMV and an argmax).  workspace: the zeroed head + 32 KiB behind it (gptq4_workspace_bytes of any operator
 * covers it).  The sums are fp32 and rounded to fp16 once, so a logit can differ from a library GEMV's by an fp16
 * ulp and the index with it where two logits are that close.  Replaces `model.lm_head(h).argmax(-1)` of a greedy
 * decoding loop (the reference's generate.py leaves both to transformers). */
int gptq4_lm_head_argmax(const void *x, const void *weight, int64_t *out, int B, int K, int V, void *workspace,
                         size_t workspace_bytes, void *stream);

/* Causal attention of S query tokens per sequence (a prompt, or a chunk of one behind `past` cached tokens): query i
 * attends to cache rows 0 .. past + i; softmax in fp32, output fp16 out [B, S, H*D] - the layout o_proj consumes, no
 * transpose.  q fp16 [B, H, S, D] (as gptq4_qkv_rotary writes it); k_cache, v_cache fp16 [B, H, kv_capacity, D] with
 * the S new tokens already in rows past .. past + S - 1 (gptq4_qkv_rotary with kv_offset = past puts them there; for
 * a plain prompt its k / v outputs serve as caches of capacity S).  D must be 128, past + S <= kv_capacity <= 2^23.  No
 * workspace.  Replaces the attention core of QuantLlamaAttention.forward for a prompt (fused_attention.py:117-141:
 * scores, causal mask, fp32 softmax, weighted sum, transpose + reshape). */
int gptq4_prefill_attention(const void *q, const void *k_cache, const void *v_cache, void *out, int B, int H, int S,
                            int D, int kv_capacity, int past, float scale, void *stream);

/* ---- Streaming-order weight layout: what the decode kernel for a handful of rows reads -------------------------
 * A decode GEMV streams every weight once; what bounds it on this GPU is how long a launch runs with nothing in
 * flight and how many separate requests a CU has to make per byte.  In streaming order the packed words of one strip
 * of 16 output columns and one unit of 128 input rows form ONE contiguous 1 KiB block in matrix-core operand order,
 * blocks ordered [strip][unit]:
 *   sweight int32 [K/8 * N]: word ((strip * K/128 + unit) * 64 + lane) * 4 + j, lane = 16 * r + c (r = 0..3, c = 0..15,
 *           j = 0..3), is qweight[(unit * 16 + 4 * r + j), strip * 16 + c] - a permutation of the words of qweight;
 *   smeta   int32 [N/16 * G * 16]: word (strip * G + g) * 16 + c = fp16 bits of scales[g, strip * 16 + c]
 *           | stored zero of that column and group << 16.
 * The kernel deals the (strip, unit) blocks of a projection evenly to one workgroup per CU, whatever the number of
 * columns, and sums inside the workgroup; only a strip that the cut between two workgroups runs through is exchanged
 * through the workspace (marked partial sums in its zero-kept head, as in the other decode kernels).  No reference
 * counterpart: the reference reads the checkpoint layout with one Triton kernel for all sizes
 * (quant_linear.py:125-225).  A load-time re-layout like gptq4_actorder_sort_rows: a caller keeps EITHER layout
 * resident (the conversion is exact both ways).  For act-order, convert the row-sorted weight and pass `perm` as to
 * the plain entry points. */

/* Most rows (M) the streaming-order entry points take for this operator and shape (at most 16); 0: the shape is not
 * supported (K below 1024, or partial sums that do not fit a CU's LDS).  Up to 4 rows the kernel keeps the rows in LDS;
 * from 5 rows on a variant fetches them with every block of weights.  `op` is a GPTQ4_OP_* matmul selector, N = I
 * for MLP_GATEUP, N = 3*H*D for QKV_ROTARY. */
int gptq4_stream_rows(int op, int K, int N, int groupsize);

/* Checkpoint order -> streaming order and back.  smeta (and with it qzeros, scales) may be NULL: words only.
 * Source and destination must not overlap. */
int gptq4_stream_pack(const int32_t *qweight, const int32_t *qzeros, const void *scales, int32_t *sweight,
                      int32_t *smeta, int K, int N, int groupsize, void *stream);
int gptq4_stream_unpack(const int32_t *sweight, const int32_t *smeta, int32_t *qweight, int32_t *qzeros,
                        void *scales, int K, int N, int groupsize, void *stream);
/* gptq4_dequant from the streaming order (row groups k / groupsize): W_out fp16 [K, N], bit-exact to the formula. */
int gptq4_stream_dequant(const int32_t *sweight, const int32_t *smeta, void *W_out, int K, int N, int groupsize,
                         void *stream);

/* gptq4_matmul / gptq4_mlp_gateup / gptq4_qkv_rotary on projections in streaming order: the decode kernels for
 * M <= gptq4_stream_rows(); for M > 16 the tiled kernel of the plain entry points, which reads the same words (a
 * shape with 0 < gptq4_stream_rows() < M <= 16: -GPTQ4_E_SHAPE).  Same arithmetic (fp16 weights of the formula above, fp32 accumulation, one rounding)
 * - only the order in which the fp32 partial sums are added differs, fixed for a shape and GPU.  The two fused
 * entry points take the residual add + RMSNorm of their input along when norm_weight is not NULL (delta, sum_out
 * as in gptq4_norm_qkv_rotary; bit-identical to gptq4_add_rmsnorm followed by the plain call; K <= 8192, M <= 4).
 * workspace: GPTQ4_WS_HEAD_BYTES, zero before the first call; a call with `perm` and more than 4 rows gathers the
 * rows into the workspace first (one small launch) and needs M * K * 2 bytes behind the head; above 16 rows
 * gptq4_workspace_bytes() of the plain operator (the tiled kernel's split-K sums). */
int gptq4_stream_matmul(const void *x, const int32_t *sweight, const int32_t *smeta, const int32_t *perm,
                        const void *bias, void *y, int M, int K, int N, int groupsize, void *workspace,
                        size_t workspace_bytes, void *stream);
int gptq4_stream_mlp_gateup(const void *x, const void *delta, const void *norm_weight, float eps, void *sum_out,
                            const int32_t *gate_sweight, const int32_t *gate_smeta, const int32_t *up_sweight,
                            const int32_t *up_smeta, const int32_t *perm, void *h, int M, int K, int I,
                            int groupsize, void *workspace, size_t workspace_bytes, void *stream);
int gptq4_stream_qkv_rotary(const void *x, const void *delta, const void *norm_weight, float eps, void *sum_out,
                            const int32_t *sweight, const int32_t *smeta, const int32_t *perm,
                            const int32_t *position_ids, const float *cos_table, const float *sin_table,
                            int max_pos, void *q, void *k, void *v, int B, int S, int H, int D, int K,
                            int groupsize, int kv_capacity, int kv_offset, void *workspace,
                            size_t workspace_bytes, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* GPTQ4_H */
