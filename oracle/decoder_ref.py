"""CPU reference for the minimal LLaMA decoder: float32 torch ops on the oracle's
dequantised weights.  TEST INFRASTRUCTURE ONLY (same rule as the rest of oracle/).

Layer structure as the reference drives it through HF's decoder layer
(fused_attention.py:79-153 for attention, fused_mlp.py:78-79 for the MLP):
x + attn(rmsnorm(x)), then h + mlp(rmsnorm(h)); rotary by the closed form in gptq_oracle.

Pinned by tests/test_oracle_transformers.py: logits equal transformers' LlamaForCausalLM (float32, the
oracle's dequantised weights loaded into its nn.Linear modules) within 1e-4; causality (logits at t do not
move when later tokens change); a model whose o_proj and down_proj decode to zero returns
lm_head(norm(embedding)).
"""
from __future__ import annotations

import math

import numpy as np
import torch

from . import gptq_oracle as O


def rmsnorm(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    return w.float() * (x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps))


def dequant(state, prefix, groupsize) -> torch.Tensor:
    g = state.get(prefix + ".g_idx")
    w = O.dequant_fp16(state[prefix + ".qweight"].numpy(), state[prefix + ".qzeros"].numpy(),
                       state[prefix + ".scales"].numpy(), groupsize, None if g is None else g.numpy())
    return torch.from_numpy(w.astype(np.float32))  # [K, N]


def forward(state: dict, cfg, groupsize: int, input_ids: torch.Tensor) -> torch.Tensor:
    """state: UNFUSED checkpoint state_dict (CPU tensors).  Returns float32 logits [B, S, V]."""
    b, s = input_ids.shape
    heads = cfg.num_attention_heads
    hd = cfg.hidden_size // heads
    cos, sin = O.rotary_tables(s, hd, cfg.rope_theta)
    cos, sin = torch.from_numpy(cos), torch.from_numpy(sin)
    h = state["model.embed_tokens.weight"].float()[input_ids]
    mask = torch.full((s, s), float("-inf")).triu(1)
    for i in range(cfg.num_hidden_layers):
        p = f"model.layers.{i}."
        x = rmsnorm(h, state[p + "input_layernorm.weight"], cfg.rms_norm_eps)
        q, k, v = (x @ dequant(state, p + f"self_attn.{n}_proj", groupsize) for n in "qkv")
        shape = lambda t: t.view(b, s, heads, hd).transpose(1, 2)
        q, k, v = shape(q), shape(k), shape(v)

        def rope(t):
            t1, t2 = t[..., :hd // 2], t[..., hd // 2:]
            return torch.cat([t1 * cos - t2 * sin, t2 * cos + t1 * sin], dim=-1)

        q, k = rope(q), rope(k)
        att = torch.softmax(q @ k.transpose(2, 3) / math.sqrt(hd) + mask, dim=-1) @ v
        h = h + att.transpose(1, 2).reshape(b, s, cfg.hidden_size) @ dequant(state, p + "self_attn.o_proj", groupsize)
        x = rmsnorm(h, state[p + "post_attention_layernorm.weight"], cfg.rms_norm_eps)
        g = x @ dequant(state, p + "mlp.gate_proj", groupsize)
        u = x @ dequant(state, p + "mlp.up_proj", groupsize)
        h = h + (torch.nn.functional.silu(g) * u) @ dequant(state, p + "mlp.down_proj", groupsize)
    h = rmsnorm(h, state["model.norm.weight"], cfg.rms_norm_eps)
    return h @ state["lm_head.weight"].float().t()
