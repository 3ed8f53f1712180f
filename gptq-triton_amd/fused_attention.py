"""Fused QKV projection + rotary embedding on the HIP kernels, and the attention module
built on it.

Mirrors src/gptq_triton/fused_attention.py of the reference: `make_quant_attn` (:10-45,
q/k/v packed tensors concatenated along N in the order q, k, v) and
`QuantLlamaAttention` (:48-153, same constructor, forward signature, return triple and
ValueErrors).  Where the reference runs one matmul, a split, three view/transposes and
the third-party rotary (:91-102), this module makes ONE call, `gptq4_qkv_rotary`, which
writes rotated Q, rotated K and V directly in [B, H, S, D].
"""
from __future__ import annotations

import math
from dataclasses import dataclass
from typing import Optional, Tuple

import torch
import torch.nn as nn

from . import _lib
from .quant_linear import (QuantLinear, _check_device_tensors, _check_matmul_args, inverse_permutation, matmul4,
                           tensor_key)


@dataclass
class LlamaConfigLite:
    """The fields of a LLaMA config this path reads."""
    hidden_size: int = 4096
    num_attention_heads: int = 32
    max_position_embeddings: int = 2048
    rope_theta: float = 10000.0
    intermediate_size: int = 11008
    num_hidden_layers: int = 32
    vocab_size: int = 32000
    rms_norm_eps: float = 1e-6


class RotaryTable:
    """cos/sin float32 [max_pos, D/2] on the device, made by gptq4_rope_table:
    angle = float32(p) * float32(base^(-2i/D)).  Stands in for the rotary_emb module
    the reference takes from its model (fused_attention.py:98-101)."""

    def __init__(self, head_dim: int, max_pos: int = 2048, base: float = 10000.0):
        self.head_dim, self.max_pos, self.base = head_dim, max_pos, float(base)
        self._tables = {}

    def get(self, device: torch.device, need_pos: int):
        key = device.index if device.index is not None else torch.cuda.current_device()
        tab = self._tables.get(key)
        if tab is None or tab[0].shape[0] < need_pos:
            n = max(self.max_pos, need_pos)
            cos = torch.empty((n, self.head_dim // 2), dtype=torch.float32, device=device)
            sin = torch.empty_like(cos)
            rc = _lib.load().gptq4_rope_table(cos.data_ptr(), sin.data_ptr(), n, self.head_dim, self.base,
                                              _lib.current_stream(device))
            _lib.check(rc, "gptq4_rope_table")
            tab = (cos, sin)
            self._tables[key] = tab
        return tab


KV_AT_POSITION = -1  # GPTQ4_KV_AT_POSITION of the C ABI


def qkv_rotary(groupsize: int, hidden_states: torch.Tensor, qweight: torch.Tensor, scales: torch.Tensor,
               qzeros: torch.Tensor, position_ids: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor,
               num_heads: int, head_dim: int = 128, perm: Optional[torch.Tensor] = None,
               kv_out: Optional[Tuple[torch.Tensor, torch.Tensor]] = None, kv_offset: int = 0, norm=None):
    """hidden_states fp16 [B, S, K]; packed weights with N = 3*H*D in q, k, v order.
    norm = (delta or None, norm_weight, eps): hidden_states is the residual stream h and the
    kernel projects RMSNorm(h + delta) * norm_weight, normalising its own input (decode-sized
    calls only, decoder_ops.norm_fusable); a fourth value is returned then, h + delta.
    Returns (q, k, v): q [B,H,S,D] rotated; k, v [B,H,S,D], or - when `kv_out` gives
    preallocated [B,H,cap,D] buffers - those buffers with rows kv_offset..kv_offset+S
    filled (kv_offset = KV_AT_POSITION: row position_ids[b, s] for token (b, s), so that a
    decode step has no host-side scalar that changes from token to token).
    position_ids int [B, S] index the cos/sin tables."""
    k_in, n = _check_matmul_args(hidden_states, qweight, groupsize)
    _check_device_tensors(hidden_states, qweight, scales, qzeros, perm, cos, sin)
    if hidden_states.dim() != 3:
        raise ValueError(f"hidden_states must be [B, S, hidden], got {tuple(hidden_states.shape)}")
    bsz, q_len, _ = hidden_states.shape
    if n != 3 * num_heads * head_dim:
        raise ValueError(f"packed QKV has {n} columns, expected 3*{num_heads}*{head_dim}")
    dev = hidden_states.device
    pos = position_ids
    if pos.dtype != torch.int32 or pos.device != dev or tuple(pos.shape) != (bsz, q_len) or not pos.is_contiguous():
        pos = position_ids.to(device=dev, dtype=torch.int32).expand(bsz, q_len).contiguous()
    q = torch.empty((bsz, num_heads, q_len, head_dim), dtype=torch.float16, device=dev)
    if kv_out is None:
        kk = torch.empty_like(q)
        vv = torch.empty_like(q)
        cap, off = q_len, 0
    else:
        kk, vv = kv_out
        cap, off = kk.shape[2], kv_offset
        if kk.shape != vv.shape or kk.shape[0] != bsz or kk.shape[1] != num_heads or kk.shape[3] != head_dim \
                or not kk.is_contiguous() or not vv.is_contiguous() or off < KV_AT_POSITION or off + q_len > cap:
            raise ValueError("kv_out buffers must be contiguous [B, H, capacity, D] with room for the new rows")
    if norm is not None:
        from .decoder_ops import check_norm_args, norm_fusable
        delta, norm_weight, eps = norm
        if not norm_fusable(bsz * q_len, k_in):
            raise ValueError("outside what the fused norm takes; run add_rms_norm and the plain call")
        h2, d2, s = check_norm_args(hidden_states, delta, norm_weight)
        lib = _lib.load()
        ws = _lib.workspace(dev, lib.gptq4_workspace_bytes(_lib.OP_QKV_ROTARY, bsz * q_len, k_in, n))
        rc = lib.gptq4_norm_qkv_rotary(h2.data_ptr(), _lib.ptr(d2), norm_weight.data_ptr(), float(eps), _lib.ptr(s),
                                       qweight.data_ptr(), qzeros.data_ptr(), scales.data_ptr(), _lib.ptr(perm), pos.data_ptr(),
                                       cos.data_ptr(), sin.data_ptr(), cos.shape[0], q.data_ptr(), kk.data_ptr(),
                                       vv.data_ptr(), bsz, q_len, num_heads, head_dim, k_in, groupsize, cap, off,
                                       ws.data_ptr(), ws.numel(), _lib.current_stream(dev))
        _lib.check(rc, "gptq4_norm_qkv_rotary")
        return q, kk, vv, (hidden_states if s is None else s.view(hidden_states.shape))
    if bsz * q_len == 0:
        return q, kk, vv
    lib = _lib.load()
    need = lib.gptq4_workspace_bytes(_lib.op_for(_lib.OP_QKV_ROTARY, perm), bsz * q_len, k_in, n)
    ws = _lib.workspace(dev, need)
    x2d = hidden_states.view(-1, k_in)
    rc = lib.gptq4_qkv_rotary(x2d.data_ptr(), qweight.data_ptr(), qzeros.data_ptr(), scales.data_ptr(),
                              _lib.ptr(perm), pos.data_ptr(), cos.data_ptr(), sin.data_ptr(), cos.shape[0],
                              q.data_ptr(), kk.data_ptr(), vv.data_ptr(), bsz, q_len, num_heads, head_dim, k_in,
                              groupsize, cap, off, ws.data_ptr(), ws.numel(), _lib.current_stream(dev))
    _lib.check(rc, "gptq4_qkv_rotary")
    return q, kk, vv


def qkv_rotary_stream(groupsize: int, hidden_states: torch.Tensor, sweight: torch.Tensor, smeta: torch.Tensor,
                      position_ids: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor, num_heads: int, head_dim: int = 128,
                      perm: Optional[torch.Tensor] = None, kv_out: Optional[Tuple[torch.Tensor, torch.Tensor]] = None,
                      kv_offset: int = 0, norm=None):
    """qkv_rotary on a projection in streaming order (quant_linear.stream_pack), for up to stream_rows() tokens in all;
    same arguments otherwise, same results to the last bit of the fp32 sums' order."""
    k_in, n = _check_matmul_args(hidden_states, sweight, groupsize)
    _check_device_tensors(hidden_states, sweight, smeta, perm, cos, sin)
    if hidden_states.dim() != 3:
        raise ValueError(f"hidden_states must be [B, S, hidden], got {tuple(hidden_states.shape)}")
    bsz, q_len, _ = hidden_states.shape
    if n != 3 * num_heads * head_dim:
        raise ValueError(f"packed QKV has {n} columns, expected 3*{num_heads}*{head_dim}")
    dev = hidden_states.device
    pos = position_ids
    if pos.dtype != torch.int32 or pos.device != dev or tuple(pos.shape) != (bsz, q_len) or not pos.is_contiguous():
        pos = position_ids.to(device=dev, dtype=torch.int32).expand(bsz, q_len).contiguous()
    q = torch.empty((bsz, num_heads, q_len, head_dim), dtype=torch.float16, device=dev)
    if kv_out is None:
        kk, vv = torch.empty_like(q), torch.empty_like(q)
        cap, off = q_len, 0
    else:
        kk, vv = kv_out
        cap, off = kk.shape[2], kv_offset
        if kk.shape != vv.shape or kk.shape[0] != bsz or kk.shape[1] != num_heads or kk.shape[3] != head_dim \
                or not kk.is_contiguous() or not vv.is_contiguous() or off < KV_AT_POSITION or off + q_len > cap:
            raise ValueError("kv_out buffers must be contiguous [B, H, capacity, D] with room for the new rows")
    delta_p = nw_p = sum_p = None
    eps, s = 0.0, None
    x2d = hidden_states.view(-1, k_in)
    if norm is not None:
        from .decoder_ops import check_norm_args
        delta, norm_weight, eps = norm
        x2d, d2, s = check_norm_args(hidden_states, delta, norm_weight)
        delta_p, nw_p, sum_p = _lib.ptr(d2), norm_weight.data_ptr(), _lib.ptr(s)
    lib = _lib.load()
    from .quant_linear import stream_workspace_bytes
    ws = _lib.workspace(dev, stream_workspace_bytes(_lib.OP_QKV_ROTARY, bsz * q_len, k_in, n, perm is not None))
    rc = lib.gptq4_stream_qkv_rotary(x2d.data_ptr(), delta_p, nw_p, float(eps), sum_p, sweight.data_ptr(), smeta.data_ptr(),
                                     _lib.ptr(perm), pos.data_ptr(), cos.data_ptr(), sin.data_ptr(), cos.shape[0], q.data_ptr(),
                                     kk.data_ptr(), vv.data_ptr(), bsz, q_len, num_heads, head_dim, k_in, groupsize, cap, off,
                                     ws.data_ptr(), ws.numel(), _lib.current_stream(dev))
    _lib.check(rc, "gptq4_stream_qkv_rotary")
    if norm is None:
        return q, kk, vv
    return q, kk, vv, (hidden_states if s is None else s.view(hidden_states.shape))


def _fuse_qkv(q_proj: QuantLinear, k_proj: QuantLinear, v_proj: QuantLinear) -> QuantLinear:
    gq, gk, gv = (getattr(p, 'g_idx', None) for p in (q_proj, k_proj, v_proj))
    have = [g is not None for g in (gq, gk, gv)]
    if any(have) and not (all(have) and torch.equal(gq.cpu(), gk.cpu()) and torch.equal(gq.cpu(), gv.cpu())):
        raise NotImplementedError("q_proj, k_proj and v_proj must share one g_idx to be fused")
    layer = QuantLinear(q_proj.bits, q_proj.groupsize, q_proj.infeatures,
                        q_proj.outfeatures + k_proj.outfeatures + v_proj.outfeatures, bias=False,
                        act_order=all(have))
    # (checkpoint_qweight: a compacted or streamed projection hands over the checkpoint's layout, not what its buffer holds)
    layer.qweight = torch.cat([q_proj.checkpoint_qweight(), k_proj.checkpoint_qweight(), v_proj.checkpoint_qweight()], dim=1)
    layer.qzeros = torch.cat([q_proj.qzeros, k_proj.qzeros, v_proj.qzeros], dim=1)
    layer.scales = torch.cat([q_proj.scales, k_proj.scales, v_proj.scales], dim=1)
    layer.bias = None
    if all(have):
        layer.g_idx = gq
    return layer


def _rope_base(config) -> float:
    """Base of the rotary embedding: `rope_theta` of the config, which newer transformers keep inside
    `rope_parameters`; only the default (unscaled) embedding is supported, as in the reference."""
    params = getattr(config, 'rope_parameters', None) or getattr(config, 'rope_scaling', None)
    if isinstance(params, dict):
        kind = params.get('rope_type', params.get('type', 'default'))
        if kind not in (None, 'default'):
            raise NotImplementedError(f"rotary embedding of type {kind!r} is not supported (only the default one)")
        if params.get('rope_theta') is not None:
            return float(params['rope_theta'])
    theta = getattr(config, 'rope_theta', None)
    return float(theta) if theta is not None else 10000.0


def _is_llama_attention(m: nn.Module) -> bool:
    if isinstance(m, QuantLlamaAttention):
        return False
    return all(isinstance(getattr(m, n, None), QuantLinear) for n in ('q_proj', 'k_proj', 'v_proj', 'o_proj'))


def make_quant_attn(model: nn.Module):
    """Replace every LLaMA attention block (q_proj/k_proj/v_proj/o_proj QuantLinears) by a
    QuantLlamaAttention with the three projections fused (fused_attention.py:10-45)."""
    for name, m in list(model.named_modules()):
        if not _is_llama_attention(m):
            continue
        if not (m.q_proj.outfeatures == m.k_proj.outfeatures == m.v_proj.outfeatures):
            raise NotImplementedError("grouped-query attention (fewer key/value heads than query heads) is not supported: "
                                      "the fused kernel takes q, k and v of one width, as the reference's does")
        qkv = _fuse_qkv(m.q_proj, m.k_proj, m.v_proj)
        attn = QuantLlamaAttention(m.config, qkv, m.o_proj, getattr(m, 'rotary_emb', None))
        attn.layer_idx = getattr(m, 'layer_idx', None)  # the slot of a transformers Cache this block updates
        parent_name, _, child = name.rpartition('.')
        parent = model.get_submodule(parent_name) if parent_name else model
        if not name:
            raise ValueError("the model itself is an attention block; wrap it in a parent module")
        setattr(parent, child, attn)


class QuantLlamaAttention(nn.Module):
    """LLaMA self-attention with the q, k, v projections and the rotary embedding fused
    into one kernel call.  Signature and return values follow the reference module."""

    def __init__(self, config, qkv_proj: QuantLinear, o_proj: QuantLinear, rotary_emb=None):
        super().__init__()
        self.config = config
        self.hidden_size = config.hidden_size
        self.num_heads = config.num_attention_heads
        self.head_dim = self.hidden_size // self.num_heads
        self.max_position_embeddings = config.max_position_embeddings
        if (self.head_dim * self.num_heads) != self.hidden_size:
            raise ValueError(
                f"hidden_size must be divisible by num_heads (got `hidden_size`: {self.hidden_size}"
                f" and `num_heads`: {self.num_heads}).")
        self.qkv_proj = qkv_proj
        self.o_proj = o_proj
        # kept for interface compatibility; the kernel reads its own table, which follows
        # the same closed form (base from config.rope_theta, default 10000)
        self.rotary_emb = rotary_emb
        self.rope = RotaryTable(self.head_dim, self.max_position_embeddings, _rope_base(config))
        self.layer_idx = None
        self._context_order = None
        self._input_order = None

    def project_qkv(self, hidden_states: torch.Tensor, position_ids: torch.Tensor,
                    kv_out=None, kv_offset: int = 0, norm=None, ordered: bool = False):
        """norm = (delta or None, norm_weight, eps): see qkv_rotary.  ordered: hidden_states already are in the
        order of input_order()."""
        # rows of the cos/sin table: with KV_AT_POSITION the positions come from the device and can be anything the
        # cache has room for, so the table covers the whole cache (the kernels clamp positions to the table)
        if kv_offset < 0 and kv_out is not None:
            need = kv_out[0].shape[2]
        else:
            need = max(kv_offset, 0) + hidden_states.shape[1]
        cos, sin = self.rope.get(hidden_states.device, max(need, self.max_position_embeddings))
        rows = hidden_states.shape[0] * hidden_states.shape[1]
        sw = self.qkv_proj.stream_weights(rows)
        from .decoder_ops import NORM_MAX_ROWS
        if sw is not None and (norm is None or rows <= NORM_MAX_ROWS):
            return qkv_rotary_stream(self.qkv_proj.groupsize, hidden_states, sw[0], sw[1], position_ids, cos, sin, self.num_heads,
                                     self.head_dim, perm=None if ordered else sw[2], kv_out=kv_out, kv_offset=kv_offset, norm=norm)
        qweight, perm = self.qkv_proj.kernel_weights()
        return qkv_rotary(self.qkv_proj.groupsize, hidden_states, qweight, self.qkv_proj.scales,
                          self.qkv_proj.qzeros, position_ids, cos, sin, self.num_heads, self.head_dim,
                          perm=None if ordered else perm, kv_out=kv_out, kv_offset=kv_offset, norm=norm)

    def context_order(self):
        """Where each feature of the attention output should be stored so that an act-order o_proj reads
        it in the order of its sorted rows (int32 [hidden], the inverse of o_proj's permutation), or
        None without act-order.  decode_attention(out_index=...) writes in that order."""
        perm = self.o_proj.row_permutation()
        if perm is None:
            return None
        if self._context_order is None or self._context_order[0] != tensor_key(perm):
            self._context_order = (tensor_key(perm), inverse_permutation(perm))
        return self._context_order[1]

    def input_order(self):
        """The same for the input of the fused QKV projection: rms_norm / add_rms_norm(out_index=...) write in
        that order, and project_qkv(ordered=True) then runs without a gather.  None without act-order."""
        perm = self.qkv_proj.row_permutation()
        if perm is None:
            return None
        if self._input_order is None or self._input_order[0] != tensor_key(perm):
            self._input_order = (tensor_key(perm), inverse_permutation(perm))
        return self._input_order[1]

    def project_out(self, context: torch.Tensor, ordered: bool = False) -> torch.Tensor:
        """o_proj(context); ordered: the context already is in the order of context_order()."""
        return self.o_proj.multiply(context, ordered=ordered)

    def norm_fusable(self, rows: int) -> bool:
        """Whether project_qkv(norm=...) is the faster way for this many rows."""
        from .decoder_ops import norm_fusion_pays
        return norm_fusion_pays(rows, self.hidden_size)

    def forward(
        self,
        hidden_states: torch.Tensor,
        attention_mask: Optional[torch.Tensor] = None,
        position_ids: Optional[torch.LongTensor] = None,
        past_key_value: Optional[Tuple[torch.Tensor]] = None,
        output_attentions: bool = False,
        use_cache: bool = False,
        past_key_values=None,
        position_embeddings=None,
        causal: bool = False,
        **kwargs,
    ) -> Tuple[torch.Tensor, Optional[torch.Tensor], Optional[Tuple[torch.Tensor]]]:
        """Input shape: Batch x Time x Channel.

        Two calling conventions.  The reference's (fused_attention.py:80-153, transformers of 2023): `past_key_value` is a
        (key, value) pair or None, the result is (output, weights or None, (key, value) or None).  Called the way the
        decoder layer of current transformers calls its attention block - `past_key_values` (a Cache object or None)
        and / or `position_embeddings` given - it updates the Cache in slot `layer_idx` and returns (output, weights or
        None); the cos / sin handed in are not used: the kernel turns q and k itself, from `position_ids`.

        causal (not in the reference, whose callers hand over an additive mask): with no attention_mask, query i attends to
        the past and to the new tokens up to itself - the prompt pass of this package's own decoder, which runs on the
        library's attention kernel instead of a materialised mask."""
        if past_key_values is not None or position_embeddings is not None:
            return self._forward_with_cache(hidden_states, attention_mask, position_ids, past_key_values,
                                            output_attentions or bool(kwargs.get('output_attentions', False)),
                                            kwargs.get('cache_position'))
        bsz, q_len, _ = hidden_states.size()
        past_len = 0 if past_key_value is None else past_key_value[0].shape[-2]
        kv_seq_len = past_len + q_len
        if position_ids is None:
            position_ids = torch.arange(past_len, kv_seq_len, device=hidden_states.device).unsqueeze(0)

        if past_key_value is None:
            query_states, key_states, value_states = self.project_qkv(hidden_states, position_ids)
        else:
            # new K/V rows are written by the kernel behind the copied past: no separate cat
            shape = (bsz, self.num_heads, kv_seq_len, self.head_dim)
            key_states = torch.empty(shape, dtype=torch.float16, device=hidden_states.device)
            value_states = torch.empty(shape, dtype=torch.float16, device=hidden_states.device)
            key_states[:, :, :past_len].copy_(past_key_value[0])
            value_states[:, :, :past_len].copy_(past_key_value[1])
            query_states, _, _ = self.project_qkv(hidden_states, position_ids,
                                                  kv_out=(key_states, value_states), kv_offset=past_len)
        past_key_value = (key_states, value_states) if use_cache else None

        if attention_mask is not None and attention_mask.size() != (bsz, 1, q_len, kv_seq_len):
            raise ValueError(
                f"Attention mask should be of size {(bsz, 1, q_len, kv_seq_len)}, but is {attention_mask.size()}")

        if causal and attention_mask is None and not output_attentions and q_len > 1 and self.head_dim == 128:
            from .decoder_ops import prefill_attention
            attn_output = prefill_attention(query_states, key_states, value_states, past_len)  # [B, S, hidden]
            return self.o_proj(attn_output), None, past_key_value
        if causal and attention_mask is None and q_len > 1:
            from .llama import causal_mask
            attention_mask = causal_mask(q_len, kv_seq_len, hidden_states.device).expand(bsz, 1, q_len, kv_seq_len)

        attn_weights = None
        if output_attentions:
            # explicit path, as the reference computes it (fused_attention.py:119-137)
            attn_weights = torch.matmul(query_states, key_states.transpose(2, 3)) / math.sqrt(self.head_dim)
            if attn_weights.size() != (bsz, self.num_heads, q_len, kv_seq_len):
                raise ValueError(
                    f"Attention weights should be of size {(bsz * self.num_heads, q_len, kv_seq_len)}, but is"
                    f" {attn_weights.size()}")
            if attention_mask is not None:
                attn_weights = attn_weights + attention_mask
                attn_weights = torch.clamp_min(attn_weights, torch.finfo(attn_weights.dtype).min)
            attn_weights = nn.functional.softmax(attn_weights, dim=-1, dtype=torch.float32).to(query_states.dtype)
            attn_output = torch.matmul(attn_weights, value_states)
        else:
            attn_output = nn.functional.scaled_dot_product_attention(
                query_states, key_states, value_states, attn_mask=attention_mask)

        if attn_output.size() != (bsz, self.num_heads, q_len, self.head_dim):
            raise ValueError(
                f"`attn_output` should be of size {(bsz, self.num_heads, q_len, self.head_dim)}, but is"
                f" {attn_output.size()}")
        attn_output = attn_output.transpose(1, 2).reshape(bsz, q_len, self.hidden_size)
        attn_output = self.o_proj(attn_output)
        return attn_output, attn_weights, past_key_value


def _forward_with_cache(self, hidden_states, attention_mask, position_ids, cache, output_attentions, cache_position):
    """The call of a current transformers decoder layer (see QuantLlamaAttention.forward)."""
    bsz, q_len, _ = hidden_states.size()
    if position_ids is None:
        if cache_position is not None:
            position_ids = cache_position.unsqueeze(0)
        else:
            past = 0 if cache is None else int(cache.get_seq_length(self.layer_idx))
            position_ids = torch.arange(past, past + q_len, device=hidden_states.device).unsqueeze(0)
    if position_ids.shape[0] != bsz:
        position_ids = position_ids.expand(bsz, -1)
    if cache is not None and self.layer_idx is None:
        raise ValueError("this attention block does not know its layer index and cannot update a Cache")
    # tokens the cache holds before this call; read only when no mask says what to attend to
    past = int(cache.get_seq_length(self.layer_idx)) if cache is not None and attention_mask is None else 0
    query_states, key_states, value_states = self.project_qkv(hidden_states, position_ids.contiguous())
    if cache is not None:
        key_states, value_states = cache.update(key_states, value_states, self.layer_idx)
    kv_len = key_states.shape[-2]
    k_all, v_all = key_states, value_states  # as the cache keeps them (a preallocated one: its whole capacity)
    if attention_mask is None and kv_len > past + q_len:
        # a preallocated cache hands back its whole capacity: without a mask only the slots written so far count
        kv_len = past + q_len
        key_states, value_states = key_states[:, :, :kv_len], value_states[:, :, :kv_len]
    causal = None
    if attention_mask is None and q_len > 1 and kv_len != q_len:
        # a prompt chunk behind cached tokens: token i sees the cached tokens and the chunk up to itself
        causal = torch.ones(q_len, kv_len, dtype=torch.bool, device=hidden_states.device).tril(kv_len - q_len)
    attn_weights = None
    if output_attentions:
        attn_weights = torch.matmul(query_states, key_states.transpose(2, 3)) / math.sqrt(self.head_dim)
        if attention_mask is not None:
            if attention_mask.dtype == torch.bool:
                attn_weights = attn_weights.masked_fill(~attention_mask[..., :kv_len], torch.finfo(attn_weights.dtype).min)
            else:
                attn_weights = torch.clamp_min(attn_weights + attention_mask[..., :kv_len], torch.finfo(attn_weights.dtype).min)
        elif q_len > 1:
            full = causal if causal is not None else torch.ones(q_len, kv_len, dtype=torch.bool, device=attn_weights.device).tril()
            attn_weights = attn_weights.masked_fill(~full, torch.finfo(attn_weights.dtype).min)
        attn_weights = nn.functional.softmax(attn_weights, dim=-1, dtype=torch.float32).to(query_states.dtype)
        attn_output = torch.matmul(attn_weights, value_states)
    elif attention_mask is None and q_len > 1 and self.head_dim == 128 and k_all.is_contiguous() and v_all.is_contiguous():
        # (the kernel reads cache rows 0 .. kv_len - 1 where they lie, whatever the capacity behind them)
        from .decoder_ops import prefill_attention
        return self.o_proj(prefill_attention(query_states, k_all, v_all, kv_len - q_len)), None
    else:
        # as transformers' own scaled-dot-product path: a given mask is used as it is, none means causal for a prompt
        # and full attention for a single token
        mask = causal if attention_mask is None else attention_mask[..., :kv_len]
        attn_output = nn.functional.scaled_dot_product_attention(query_states, key_states, value_states, attn_mask=mask,
                                                                 is_causal=(mask is None and q_len > 1))
    attn_output = attn_output.transpose(1, 2).reshape(bsz, q_len, self.hidden_size)
    return self.o_proj(attn_output), attn_weights


QuantLlamaAttention._forward_with_cache = _forward_with_cache
