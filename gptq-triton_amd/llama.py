"""A minimal LLaMA decoder around the quantised hot path.

The reference builds an un-initialised HF `LlamaForCausalLM` and swaps modules in it
(src/gptq_triton/__init__.py:32-77); generation is then HF's (generate.py:41-50).  Here the
model skeleton is a few lines of plain torch with the same module tree and therefore the
same state_dict keys (`model.layers.{i}.self_attn.q_proj.qweight`, ...), so reference
checkpoints load unchanged and nothing depends on transformers at run time.  RMSNorm,
residuals, the attention core and the fp16 lm_head are torch ops; every linear inside the
layers is the HIP path.
"""
from __future__ import annotations

import json
from pathlib import Path
from typing import List, Optional, Tuple

import torch
import torch.nn as nn

from .fused_attention import LlamaConfigLite


def config_from_json(path) -> LlamaConfigLite:
    """Read the fields this path needs from an HF-style config.json."""
    raw = json.load(open(path))
    cfg = LlamaConfigLite()
    for field in ("hidden_size", "num_attention_heads", "max_position_embeddings", "rope_theta", "intermediate_size",
                  "num_hidden_layers", "vocab_size", "rms_norm_eps"):
        if field in raw:
            setattr(cfg, field, raw[field])
    kv = raw.get("num_key_value_heads", cfg.num_attention_heads)
    if kv != cfg.num_attention_heads:
        raise NotImplementedError("grouped-query attention is outside the LLaMA-1 family this path covers")
    return cfg


class LlamaRMSNorm(nn.Module):
    def __init__(self, hidden_size: int, eps: float = 1e-6):
        super().__init__()
        self.weight = nn.Parameter(torch.ones(hidden_size, dtype=torch.float16), requires_grad=False)
        self.variance_epsilon = eps

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        xf = x.float()
        xf = xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + self.variance_epsilon)
        return self.weight * xf.to(x.dtype)


class LlamaAttention(nn.Module):
    """Skeleton attention block: four linears to be replaced by make_quant / make_quant_attn."""

    def __init__(self, config):
        super().__init__()
        self.config = config
        h = config.hidden_size
        self.q_proj = nn.Linear(h, h, bias=False)
        self.k_proj = nn.Linear(h, h, bias=False)
        self.v_proj = nn.Linear(h, h, bias=False)
        self.o_proj = nn.Linear(h, h, bias=False)


class LlamaMLP(nn.Module):
    """Skeleton MLP block: three linears to be replaced by make_quant / make_fused_mlp."""

    def __init__(self, config):
        super().__init__()
        h, i = config.hidden_size, config.intermediate_size
        self.gate_proj = nn.Linear(h, i, bias=False)
        self.down_proj = nn.Linear(i, h, bias=False)
        self.up_proj = nn.Linear(h, i, bias=False)

    def forward(self, x):  # unfused path: three QuantLinear calls + torch silu*mul
        return self.down_proj(torch.nn.functional.silu(self.gate_proj(x)) * self.up_proj(x))


class LlamaDecoderLayer(nn.Module):
    def __init__(self, config):
        super().__init__()
        self.self_attn = LlamaAttention(config)
        self.mlp = LlamaMLP(config)
        self.input_layernorm = LlamaRMSNorm(config.hidden_size, config.rms_norm_eps)
        self.post_attention_layernorm = LlamaRMSNorm(config.hidden_size, config.rms_norm_eps)

    def forward(self, hidden_states, attention_mask=None, position_ids=None, past_key_value=None, use_cache=False):
        attn_out, _, present = self.self_attn(hidden_states=self.input_layernorm(hidden_states),
                                              attention_mask=attention_mask, position_ids=position_ids,
                                              past_key_value=past_key_value, use_cache=use_cache)
        hidden_states = hidden_states + attn_out
        hidden_states = hidden_states + self.mlp(self.post_attention_layernorm(hidden_states))
        return hidden_states, present


class LlamaModel(nn.Module):
    def __init__(self, config):
        super().__init__()
        self.embed_tokens = nn.Embedding(config.vocab_size, config.hidden_size)
        self.layers = nn.ModuleList([LlamaDecoderLayer(config) for _ in range(config.num_hidden_layers)])
        self.norm = LlamaRMSNorm(config.hidden_size, config.rms_norm_eps)


def causal_mask(q_len: int, kv_len: int, device, dtype=torch.float16) -> Optional[torch.Tensor]:
    """Additive [1, 1, q_len, kv_len] mask; None when a single query row sees everything."""
    if q_len == 1:
        return None
    past = kv_len - q_len
    i = torch.arange(q_len, device=device)[:, None]
    j = torch.arange(kv_len, device=device)[None, :]
    m = torch.zeros((q_len, kv_len), dtype=dtype, device=device)
    m.masked_fill_(j > i + past, torch.finfo(dtype).min)
    return m[None, None]


class LlamaForCausalLM(nn.Module):
    def __init__(self, config):
        super().__init__()
        self.config = config
        self.model = LlamaModel(config)
        self.lm_head = nn.Linear(config.hidden_size, config.vocab_size, bias=False)
        self.seqlen = config.max_position_embeddings

    @torch.no_grad()
    def forward(self, input_ids: torch.Tensor, past_key_values: Optional[List[Tuple[torch.Tensor, torch.Tensor]]] = None,
                use_cache: bool = False, last_token_only: bool = False):
        """input_ids [B, S] -> (logits [B, S or 1, vocab], past_key_values or None)."""
        bsz, q_len = input_ids.shape
        past_len = 0 if past_key_values is None else past_key_values[0][0].shape[2]
        position_ids = torch.arange(past_len, past_len + q_len, device=input_ids.device).unsqueeze(0)
        mask = causal_mask(q_len, past_len + q_len, input_ids.device)
        if mask is not None:
            mask = mask.expand(bsz, 1, q_len, past_len + q_len)
        h = self.model.embed_tokens(input_ids)
        presents = []
        for i, layer in enumerate(self.model.layers):
            h, present = layer(h, attention_mask=mask, position_ids=position_ids,
                               past_key_value=None if past_key_values is None else past_key_values[i], use_cache=use_cache)
            presents.append(present)
        h = self.model.norm(h)
        if last_token_only:
            h = h[:, -1:, :]
        return self.lm_head(h), (presents if use_cache else None)

    @torch.no_grad()
    def generate_greedy(self, input_ids: torch.Tensor, max_new_tokens: int) -> torch.Tensor:
        """Prefill + greedy decode with a preallocated KV cache: the fused QKV kernel writes
        rotated K and V straight into the cache (no cat, no copies)."""
        bsz, prompt = input_ids.shape
        dev = input_ids.device
        cfg = self.config
        heads, hd = cfg.num_attention_heads, cfg.hidden_size // cfg.num_attention_heads
        cap = prompt + max_new_tokens
        caches = [(torch.empty((bsz, heads, cap, hd), dtype=torch.float16, device=dev),
                   torch.empty((bsz, heads, cap, hd), dtype=torch.float16, device=dev)) for _ in self.model.layers]
        out = [input_ids]
        tokens, cur = input_ids, 0
        for step in range(max_new_tokens):
            q_len = tokens.shape[1]
            position_ids = torch.arange(cur, cur + q_len, device=dev).unsqueeze(0)
            mask = causal_mask(q_len, cur + q_len, dev)
            h = self.model.embed_tokens(tokens)
            for layer, (kc, vc) in zip(self.model.layers, caches):
                x = layer.input_layernorm(h)
                attn = layer.self_attn
                q, _, _ = attn.project_qkv(x, position_ids, kv_out=(kc, vc), kv_offset=cur)
                o = torch.nn.functional.scaled_dot_product_attention(q, kc[:, :, :cur + q_len], vc[:, :, :cur + q_len],
                                                                     attn_mask=mask)
                h = h + attn.o_proj(o.transpose(1, 2).reshape(bsz, q_len, cfg.hidden_size))
                h = h + layer.mlp(layer.post_attention_layernorm(h))
            logits = self.lm_head(self.model.norm(h[:, -1:, :]))
            tokens = logits.argmax(-1)
            out.append(tokens)
            cur += q_len
        return torch.cat(out, dim=1)
