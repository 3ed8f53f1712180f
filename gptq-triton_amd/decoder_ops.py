"""The two non-matmul operators of a decode step, as HIP kernels behind the C ABI: RMSNorm
and single-query attention over a preallocated KV cache.  The reference runs both as torch
ops of the HF model it patches (LlamaRMSNorm; fused_attention.py:118-148); here they exist
so that a whole decode step is a short chain of HIP launches that a graph can replay."""
from __future__ import annotations

import math
import os

import torch

from . import _lib


# limits of the matmul kernels that normalise their own input (gptq4_norm_qkv_rotary, gptq4_norm_mlp_gateup)
NORM_MAX_ROWS, NORM_MAX_HIDDEN = 4, 8192
# up to how many rows the decoder uses them: one row costs 1.3-1.4 us on top of the plain projection against
# a 4.7 us norm launch; two rows about as much as the launch, three and four more (every workgroup
# normalises every row)
NORM_PAYS_ROWS = 1
# GPTQ4_NORM_FUSION=0 in the environment keeps the norms as launches of their own (for A/B timing)
NORM_FUSION = os.environ.get("GPTQ4_NORM_FUSION", "1") != "0"


def norm_fusable(rows: int, hidden: int) -> bool:
    """Whether a projection of `rows` rows CAN take the residual add + RMSNorm of its input along."""
    return 0 < rows <= NORM_MAX_ROWS and hidden <= NORM_MAX_HIDDEN and hidden % 8 == 0


def norm_fusion_pays(rows: int, hidden: int) -> bool:
    """Whether it is also the faster way (what the decoder asks)."""
    return NORM_FUSION and rows <= NORM_PAYS_ROWS and norm_fusable(rows, hidden)


def check_norm_args(h: torch.Tensor, delta, weight: torch.Tensor):
    """Validate (h, delta, norm weight) of a fused call; returns the [rows, hidden] views and the sum buffer."""
    for t, name in ((h, "h"), (delta, "delta"), (weight, "norm weight")):
        if t is None:
            continue
        _lib.require_cuda(t, name)
        if t.dtype != torch.float16:
            raise TypeError("the fused residual add + RMSNorm takes fp16 tensors")
    hidden = h.shape[-1]
    if weight.shape != (hidden,) or (delta is not None and delta.shape != h.shape):
        raise ValueError("h and delta must have one shape [..., H] and the norm weight [H]")
    h2 = h.reshape(-1, hidden).contiguous()
    d2 = None if delta is None else delta.reshape(-1, hidden).contiguous()
    s = None if delta is None else torch.empty_like(h2)  # never aliases h or delta: other workgroups still read them
    return h2, d2, s


def _check_out_index(out_index, h: int) -> None:
    if out_index is not None:
        _lib.require_cuda(out_index, "out_index")
        if out_index.dtype != torch.int32 or out_index.shape != (h,) or not out_index.is_contiguous():
            raise ValueError(f"out_index must be a contiguous int32 tensor of {h} positions")


def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float, out_index: torch.Tensor = None) -> torch.Tensor:
    """y = weight * fp16(x * rsqrt(mean(x^2, -1) + eps)) for fp16 x [..., H] on the GPU.  With out_index (int32
    [H], a permutation) value f of a row is stored at position out_index[f]."""
    _lib.require_cuda(x, "x")
    _lib.require_cuda(weight, "weight")
    if x.dtype != torch.float16 or weight.dtype != torch.float16:
        raise TypeError("rms_norm takes fp16 tensors")
    h = x.shape[-1]
    if weight.shape != (h,) or h % 8 != 0:
        raise ValueError(f"weight must be [{h}] and the hidden size a multiple of 8")
    _check_out_index(out_index, h)
    x2 = x.reshape(-1, h)
    if not x2.is_contiguous():
        x2 = x2.contiguous()
    y = torch.empty_like(x2)
    if x2.shape[0] == 0:
        return y.reshape(x.shape)
    rc = _lib.load().gptq4_rmsnorm(x2.data_ptr(), weight.data_ptr(), y.data_ptr(), _lib.ptr(out_index), x2.shape[0], h,
                                   float(eps), _lib.current_stream(x.device))
    _lib.check(rc, "gptq4_rmsnorm")
    return y.reshape(x.shape)


def add_rms_norm(x: torch.Tensor, delta: torch.Tensor, weight: torch.Tensor, eps: float, out_index: torch.Tensor = None):
    """(x + delta, RMSNorm(x + delta)) in one launch; fp16 GPU tensors of equal shape [..., H].  out_index as in
    rms_norm (the sum keeps its order)."""
    for t, name in ((x, "x"), (delta, "delta"), (weight, "weight")):
        _lib.require_cuda(t, name)
        if t.dtype != torch.float16:
            raise TypeError("add_rms_norm takes fp16 tensors")
    h = x.shape[-1]
    if delta.shape != x.shape or weight.shape != (h,) or h % 8 != 0:
        raise ValueError("x and delta must have one shape [..., H], weight [H], H a multiple of 8")
    _check_out_index(out_index, h)
    x2 = x.reshape(-1, h).contiguous()
    d2 = delta.reshape(-1, h).contiguous()
    s = torch.empty_like(x2)
    y = torch.empty_like(x2)
    if x2.shape[0]:
        rc = _lib.load().gptq4_add_rmsnorm(x2.data_ptr(), d2.data_ptr(), weight.data_ptr(), s.data_ptr(), y.data_ptr(),
                                           _lib.ptr(out_index), x2.shape[0], h, float(eps), _lib.current_stream(x.device))
        _lib.check(rc, "gptq4_add_rmsnorm")
    return s.reshape(x.shape), y.reshape(x.shape)


HEAD_ARGMAX_K = (4096, 5120, 6656, 8192)  # row lengths gptq4_lm_head_argmax is built for


def lm_head_argmax(x: torch.Tensor, weight: torch.Tensor, max_rows: int = 4) -> torch.Tensor:
    """Greedy next tokens: argmax(x @ weight.T, -1) in one launch, for x fp16 [..., K] and an fp16 lm_head weight [V, K].
    Returns int64 of x's shape without the last dimension.  The kernel takes up to 16 rows but pays up to `max_rows`
    (one row of 4096: 52 us against 77 for the library's GEMV + argmax; eight rows: 97 against 83); more rows, and shapes
    it is not built for, go through torch."""
    k = x.shape[-1]
    rows = x.numel() // max(k, 1)
    if not (x.is_cuda and x.dtype == torch.float16 and weight.dtype == torch.float16 and weight.is_contiguous() and weight.dim() == 2
            and weight.shape[1] == k and k in HEAD_ARGMAX_K and 0 < rows <= min(max_rows, 16) and rows * k * 2 <= 160 * 1024 - 2048
            and weight.numel() * 2 < 0x7FFFFFF0):
        return torch.nn.functional.linear(x, weight).argmax(-1)
    xc = x.reshape(rows, k).contiguous()
    out = torch.empty(rows, dtype=torch.int64, device=x.device)
    ws = _lib.workspace(x.device, _lib.WS_HEAD_BYTES + (64 << 10))
    rc = _lib.load().gptq4_lm_head_argmax(xc.data_ptr(), weight.data_ptr(), out.data_ptr(), rows, k, weight.shape[0], ws.data_ptr(), ws.numel(),
                                          _lib.current_stream(x.device))
    _lib.check(rc, "gptq4_lm_head_argmax")
    return out.view(x.shape[:-1])


def prefill_attention(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, past: int = 0) -> torch.Tensor:
    """Causal attention of a prompt (or of a chunk behind `past` cached tokens): q fp16 [B, H, S, 128]; caches fp16
    [B, H, capacity, 128] holding the S new tokens in rows past .. past + S - 1 (for a plain prompt: the k and v the QKV
    projection returned); query i attends to rows 0 .. past + i.  Returns fp16 [B, S, H*128], what o_proj consumes."""
    for t, name in ((q, "q"), (k_cache, "k_cache"), (v_cache, "v_cache")):
        _lib.require_cuda(t, name)
        if t.dtype != torch.float16:
            raise TypeError("prefill_attention takes fp16 tensors")
    bsz, heads, q_len, hd = q.shape
    if hd != 128:
        raise ValueError("prefill_attention needs head_dim 128")
    if k_cache.shape != v_cache.shape or k_cache.shape[:2] != (bsz, heads) or k_cache.shape[3] != hd \
            or not (q.is_contiguous() and k_cache.is_contiguous() and v_cache.is_contiguous()):
        raise ValueError("caches must be contiguous [B, H, capacity, 128] tensors matching q")
    cap = k_cache.shape[2]
    if past < 0 or past + q_len > cap:
        raise ValueError("the cache has no room for past + S rows")
    out = torch.empty((bsz, q_len, heads * hd), dtype=torch.float16, device=q.device)
    if q_len:
        rc = _lib.load().gptq4_prefill_attention(q.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(), out.data_ptr(), bsz, heads, q_len,
                                                 hd, cap, past, 1.0 / math.sqrt(hd), _lib.current_stream(q.device))
        _lib.check(rc, "gptq4_prefill_attention")
    return out


def decode_attention(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, positions: torch.Tensor,
                     out_index: torch.Tensor = None) -> torch.Tensor:
    """q fp16 [B, H, 1, 128]; caches fp16 [B, H, capacity, 128]; positions int32 [B] or [B, 1]:
    sequence b attends to cache rows 0..positions[b].  Returns fp16 [B, 1, H*128]; with out_index
    (int32 [H*128], a permutation) feature f of a row is stored at position out_index[f]."""
    for t, name in ((q, "q"), (k_cache, "k_cache"), (v_cache, "v_cache"), (positions, "positions")):
        _lib.require_cuda(t, name)
    bsz, heads, q_len, hd = q.shape
    if q_len != 1 or hd != 128:
        raise ValueError("decode_attention takes one query token per sequence and head_dim 128")
    if k_cache.shape != v_cache.shape or k_cache.shape[:2] != (bsz, heads) or k_cache.shape[3] != hd \
            or not (q.is_contiguous() and k_cache.is_contiguous() and v_cache.is_contiguous()):
        raise ValueError("caches must be contiguous [B, H, capacity, 128] tensors matching q")
    if q.dtype != torch.float16 or k_cache.dtype != torch.float16 or v_cache.dtype != torch.float16:
        raise TypeError("decode_attention takes fp16 tensors")
    pos = positions.reshape(-1)
    if pos.dtype != torch.int32 or pos.numel() != bsz or not pos.is_contiguous():
        pos = pos.to(torch.int32).contiguous()
        if pos.numel() != bsz:
            raise ValueError("one position per sequence")
    _check_out_index(out_index, heads * hd)
    cap = k_cache.shape[2]
    out = torch.empty((bsz, 1, heads * hd), dtype=torch.float16, device=q.device)
    lib = _lib.load()
    ws = _lib.workspace(q.device, lib.gptq4_workspace_bytes(_lib.OP_DECODE_ATTENTION, bsz * heads, cap, 0))
    rc = lib.gptq4_decode_attention(q.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(), pos.data_ptr(), out.data_ptr(),
                                    _lib.ptr(out_index), bsz, heads, hd, cap, 1.0 / math.sqrt(hd), ws.data_ptr(), ws.numel(),
                                    _lib.current_stream(q.device))
    _lib.check(rc, "gptq4_decode_attention")
    return out
