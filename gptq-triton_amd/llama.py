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

from . import _lib
from .decoder_ops import add_rms_norm, decode_attention, lm_head_argmax, rms_norm
from .fused_attention import LlamaConfigLite

# up to this many rows the decoder's norms write act-order inputs in their consumer's order
ORDERED_NORM_ROWS = 16
# the rows the decode kernels built on the streaming-order weight layout take (more rows: the mid-M and tiled kernels)
STREAM_BATCH = 16


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
        if x.is_cuda and x.dtype == torch.float16:
            return rms_norm(x, self.weight, self.variance_epsilon)  # one HIP launch
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

    def forward(self, hidden_states, attention_mask=None, position_ids=None, past_key_value=None, use_cache=False, causal=False):
        attn_out, _, present = self.self_attn(hidden_states=self.input_layernorm(hidden_states),
                                              attention_mask=attention_mask, position_ids=position_ids,
                                              past_key_value=past_key_value, use_cache=use_cache, causal=causal)
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
        h = self.model.embed_tokens(input_ids)
        presents = []
        for i, layer in enumerate(self.model.layers):
            # (causal: the attention block masks by position itself - on the GPU inside the attention kernel)
            h, present = layer(h, attention_mask=None, position_ids=position_ids,
                               past_key_value=None if past_key_values is None else past_key_values[i], use_cache=use_cache,
                               causal=True)
            presents.append(present)
        h = self.model.norm(h)
        if last_token_only:
            h = h[:, -1:, :]
        return self.lm_head(h), (presents if use_cache else None)

    @torch.no_grad()
    def generate_greedy(self, input_ids: torch.Tensor, max_new_tokens: int, use_graph: bool = False) -> torch.Tensor:
        """Prefill + greedy decode with a preallocated KV cache: the fused QKV kernel writes
        rotated K and V straight into the cache (no cat, no copies).  use_graph replays one
        captured HIP graph per decode token instead of launching the step's kernels one by
        one."""
        bsz, prompt = input_ids.shape
        dec = GreedyDecoder(self, bsz, prompt + max_new_tokens)
        first = dec.prefill(input_ids)
        rest = dec.decode(max_new_tokens - 1, use_graph=use_graph) if max_new_tokens > 1 else first[:, :0]
        return torch.cat([input_ids, first, rest], dim=1)


class GreedyDecoder:
    """Greedy generation state for one batch: KV caches of fixed capacity plus the static
    token / position buffers a decode step reads and writes.  Nothing in a decode step
    depends on a host-side value that changes from token to token (the QKV kernel places
    K and V by position id, the attention kernel reads how far to attend from the position
    buffer), so the step can be captured once as a HIP graph and replayed."""

    def __init__(self, model: LlamaForCausalLM, bsz: int, capacity: int, layout: str = 'auto'):
        """layout: 'stream' / 'checkpoint' put the model's packed weights into that layout first (quant_linear.set_layout;
        one copy either way), 'keep' leaves them as they are, 'auto' = 'stream': every kernel reads that layout, and the
        decode kernels for up to STREAM_BATCH rows are built on it."""
        cfg = model.config
        self.model, self.bsz, self.capacity = model, bsz, capacity
        dev = model.lm_head.weight.device
        if layout == 'auto':
            layout = 'stream'
        if layout != 'keep' and dev.type == 'cuda':
            from .quant_linear import set_layout
            set_layout(model, layout)
        heads, hd = cfg.num_attention_heads, cfg.hidden_size // cfg.num_attention_heads
        self.caches = [(torch.zeros((bsz, heads, capacity, hd), dtype=torch.float16, device=dev),
                        torch.zeros((bsz, heads, capacity, hd), dtype=torch.float16, device=dev))
                       for _ in model.model.layers]
        self.tokens = torch.zeros((bsz, 1), dtype=torch.long, device=dev)
        self.position = torch.zeros((bsz, 1), dtype=torch.int32, device=dev)
        self.graph = None

    def _layers(self, h, position_ids, kv_offset, attend):
        """The decoder stack on hidden states h [B, S, hidden]; every residual add is fused
        with the RMSNorm that follows it.  Returns the greedy next token [B, 1]."""
        layers = self.model.model.layers
        rows = h.shape[0] * h.shape[1]
        if all(getattr(l.self_attn, "norm_fusable", lambda r: False)(rows) and getattr(l.mlp, "norm_fusable", lambda r: False)(rows)
               for l in layers):
            return self._layers_norm_in_matmul(h, position_ids, kv_offset, attend)
        # act-order and a handful of rows: every norm writes in the order its consumer's sorted rows read, so the
        # consumer needs no gather launch (tall inputs leave the gather to the consumer: there the norm's
        # scattered 2-byte stores would cost more than the copy)
        def order_of(block):
            fn = getattr(block, "input_order", None)
            return fn() if fn is not None and rows <= ORDERED_NORM_ROWS else None

        n0 = layers[0].input_layernorm
        oq = order_of(layers[0].self_attn)
        x = rms_norm(h, n0.weight, n0.variance_epsilon, out_index=oq)
        for i, (layer, (kc, vc)) in enumerate(zip(layers, self.caches)):
            attn = layer.self_attn
            q, _, _ = attn.project_qkv(x, position_ids, kv_out=(kc, vc), kv_offset=kv_offset, ordered=oq is not None)
            norm = layer.post_attention_layernorm
            om = order_of(layer.mlp)
            # attend -> ([B, S, hidden], whether in attn.context_order())
            h, x = add_rms_norm(h, attn.project_out(*attend(q, kc, vc, attn)), norm.weight, norm.variance_epsilon, out_index=om)
            last = i + 1 == len(layers)
            norm = self.model.model.norm if last else layers[i + 1].input_layernorm
            oq = None if last else order_of(layers[i + 1].self_attn)
            y = layer.mlp(x, ordered=True) if om is not None else layer.mlp(x)
            h, x = add_rms_norm(h, y, norm.weight, norm.variance_epsilon, out_index=oq)
        return lm_head_argmax(x[:, -1:, :], self.model.lm_head.weight)

    def _layers_norm_in_matmul(self, h, position_ids, kv_offset, attend):
        """The same stack for a handful of rows: the QKV and the gate/up launch each do the residual
        add and the RMSNorm of their own input (same bits as _layers' separate launches), so a
        layer is 5 launches instead of 7."""
        layers = self.model.model.layers
        delta = None
        for layer, (kc, vc) in zip(layers, self.caches):
            attn, n1, n2 = layer.self_attn, layer.input_layernorm, layer.post_attention_layernorm
            q, _, _, h = attn.project_qkv(h, position_ids, kv_out=(kc, vc), kv_offset=kv_offset,
                                          norm=(delta, n1.weight, n1.variance_epsilon))
            h, delta = layer.mlp.forward_normed(h, attn.project_out(*attend(q, kc, vc, attn)), n2.weight, n2.variance_epsilon)
        norm = self.model.model.norm
        h, x = add_rms_norm(h, delta, norm.weight, norm.variance_epsilon)
        return lm_head_argmax(x[:, -1:, :], self.model.lm_head.weight)

    @torch.no_grad()
    def prefill(self, input_ids: torch.Tensor) -> torch.Tensor:
        """Run the prompt (positions 0..S-1), fill the caches, return the first new token [B, 1]."""
        bsz, prompt = input_ids.shape
        if bsz != self.bsz or prompt >= self.capacity:
            raise ValueError("prompt does not fit this decoder's batch size / capacity")
        dev = input_ids.device
        position_ids = torch.arange(prompt, device=dev, dtype=torch.int32).unsqueeze(0).expand(bsz, prompt).contiguous()
        from .decoder_ops import prefill_attention

        def attend(q, kc, vc, attn):
            # the prompt's K and V are in cache rows 0 .. prompt - 1 already; the result comes in o_proj's input layout
            return prefill_attention(q, kc, vc, 0), False

        nxt = self._layers(self.model.model.embed_tokens(input_ids), position_ids, 0, attend)
        self.tokens.copy_(nxt)
        self.position.fill_(prompt)
        return nxt

    def _step(self):
        """One decode token from the static buffers: reads tokens/position, writes them back."""
        from .fused_attention import KV_AT_POSITION

        def attend(q, kc, vc, attn):  # rows 0..position of the cache; act-order o_proj: written in the order it reads
            order = attn.context_order()
            return decode_attention(q, kc, vc, self.position, out_index=order), order is not None

        nxt = self._layers(self.model.model.embed_tokens(self.tokens), self.position, KV_AT_POSITION, attend)
        self.tokens.copy_(nxt)
        self.position.add_(1)

    @torch.no_grad()
    def decode(self, steps: int, use_graph: bool = False) -> torch.Tensor:
        """`steps` more greedy tokens after prefill -> [B, steps]."""
        out = torch.empty((self.bsz, steps), dtype=torch.long, device=self.tokens.device)
        if int(self.position.max()) + steps > self.capacity:
            raise ValueError("decode would run past the cache capacity")
        if use_graph and self.graph is None and steps > 0:
            self._capture()
        for i in range(steps):
            if use_graph:
                self.graph.replay()
            else:
                self._step()
            out[:, i:i + 1].copy_(self.tokens)
        # one 4-byte read per workspace: a bounded wait of the small-M kernels that ran out would have made tokens wrong silently
        _lib.check_exchange_errors()
        return out

    def _capture(self):
        """Capture _step as a graph.  The warm-up steps run on the capture stream first, so
        workspaces and tables exist before capture; their effect on tokens, position and the
        cache rows they wrote is undone (the rows lie beyond the current position and are
        rewritten before any later step attends to them)."""
        tokens0, position0 = self.tokens.clone(), self.position.clone()
        side = torch.cuda.Stream(device=self.tokens.device)
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            self._step()
            self.tokens.copy_(tokens0)
            self.position.copy_(position0)
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        self.graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(self.graph, stream=side):
            self._step()
        self.tokens.copy_(tokens0)
        self.position.copy_(position0)
        torch.cuda.synchronize()
