"""Checkpoint loading and saving in the reference's format.

A checkpoint directory holds `quant_config.json` ({"wbits", "groupsize"}), an HF-style
`config.json` and `model.safetensors` or `model.pt` with the UNFUSED per-projection tensors
(quantize.py:62-79).  `load_quant` follows src/gptq_triton/__init__.py:16-93 step by step:
build the skeleton, make_quant, load_state_dict, drop all-zero biases, fuse QKV, fuse the MLP
(by default only without grouping, as the reference does), move to the device.
"""
from __future__ import annotations

import json
from pathlib import Path
from typing import Optional

import torch

from . import _lib, fused_mlp, quant_linear
from .fused_attention import make_quant_attn
from .fused_mlp import make_fused_mlp
from .llama import LlamaForCausalLM, config_from_json
from .quant_linear import QuantLinear, make_quant


def load_quant(checkpoint: str, warmup_autotune: bool = True, device: Optional[str] = 'cuda',
               fuse_mlp: Optional[bool] = None, use_transformers: bool = False, compact: bool = True,
               layout: str = 'stream'):
    """Load a quantised model from a checkpoint directory.

    use_transformers: build the skeleton as the reference does (src/gptq_triton/__init__.py:32-52): a
    `transformers.LlamaForCausalLM` from the checkpoint's config.json, whose linears, attention blocks and MLPs are
    then replaced - the result is a transformers model (`generate`, Cache objects, pipelines).  Default: this
    package's own minimal decoder, which needs no transformers at run time.

    compact: act-order checkpoints on a GPU keep ONE copy of every packed weight, in the layout the kernels read
    (QuantLinear.compact, QuantLlamaMLP.compact); state_dict() / save_quant() still produce the checkpoint layout.
    With False the kernel layout is built at first use beside the checkpoint tensors (twice the weight memory).

    layout: 'stream' (default; GPU only) keeps every packed weight in streaming order, the layout the decode kernels for
    up to sixteen rows are built on (quant_linear.set_layout, QuantLinear.to_stream) - one copy of the weights either
    way, and state_dict() / save_quant() produce the checkpoint layout.  Calls with more rows (a prompt pass) read the
    same words with the mid-M and the tiled kernel, at the speed they read the checkpoint layout.  'checkpoint' keeps
    the file's layout (what the functional API on raw checkpoint tensors computes on; its decode kernels for up to
    sixteen rows are the slower ones).

    warmup_autotune is accepted for compatibility: launch shapes are static, there is
    nothing to tune (the reference spends 18-49 s here).  It still requires a device, as
    the reference does.  fuse_mlp None = fuse only when the model has no grouping.
    """
    ckpt = Path(checkpoint)
    quant_config = json.load(open(ckpt / 'quant_config.json'))
    wbits, groupsize = quant_config['wbits'], quant_config['groupsize']
    config = config_from_json(ckpt / 'config.json')

    default_dtype = torch.get_default_dtype()
    torch.set_default_dtype(torch.half)
    try:
        with torch.device('meta'):
            if use_transformers:
                import transformers
                hf_config = transformers.LlamaConfig.from_pretrained(str(ckpt))
                model = transformers.LlamaForCausalLM(hf_config)
            else:
                model = LlamaForCausalLM(config)
    finally:
        torch.set_default_dtype(default_dtype)
    model = model.to_empty(device='cpu')
    if use_transformers:
        # buffers that are computed, not stored (the rotary frequencies), are lost on the meta device: rebuild their modules
        for name, m in list(model.named_modules()):
            if name and any(b == 'inv_freq' for b, _ in m.named_buffers(recurse=False)):
                parent_name, _, child = name.rpartition('.')
                parent = model.get_submodule(parent_name) if parent_name else model
                setattr(parent, child, type(m)(config=hf_config))

    if (ckpt / 'model.safetensors').exists():
        from safetensors.torch import load_file
        state = load_file(str(ckpt / 'model.safetensors'))
    elif (ckpt / 'model.pt').exists():
        state = torch.load(ckpt / 'model.pt', weights_only=True)
    else:
        raise FileNotFoundError(f"Could not find model checkpoint at {checkpoint}; please ensure that the path is "
                                "correct and contains a `model.pt` or `model.safetensors` file.")
    act_order = any(k.endswith('.g_idx') for k in state)
    make_quant(model, wbits, groupsize, act_order=act_order)
    # rotary tables are recomputed, not loaded
    state = {k: v for k, v in state.items() if not k.endswith('rotary_emb.inv_freq')}
    # a checkpoint may carry biases for projections whose skeleton linear has none
    for key in state:
        if key.endswith('.bias'):
            m = model.get_submodule(key[:-len('.bias')])
            if isinstance(m, QuantLinear) and m.bias is None:
                del m._parameters['bias']
                m.register_buffer('bias', torch.empty(m.outfeatures, dtype=torch.float16))
    missing, unexpected = model.load_state_dict(state, strict=False)
    missing = [k for k in missing if not k.endswith('.bias')]
    if missing or unexpected:
        raise RuntimeError(f"checkpoint does not match the model: missing {missing[:5]}, unexpected {unexpected[:5]}")

    for _, m in model.named_modules():
        if isinstance(m, QuantLinear) and m.bias is not None and bool((m.bias == 0).all()):
            m.bias = None

    make_quant_attn(model)
    if fuse_mlp is True or (fuse_mlp is None and groupsize == -1):
        make_fused_mlp(model)

    if device is not None:
        model = model.to(device)
        if compact and act_order and torch.device(device).type == 'cuda':
            quant_linear.compact_act_order(model)
        if layout == 'stream' and torch.device(device).type == 'cuda':
            quant_linear.set_layout(model, 'stream')
        elif layout not in ('stream', 'checkpoint'):
            raise ValueError("layout must be 'stream' or 'checkpoint'")
    if warmup_autotune:
        if device is None:
            raise ValueError("You must specify a device when warmup_autotune is True.")
        autotune_warmup(model)
    model.seqlen = 2048
    if use_transformers and device is not None and torch.device(device).type == 'cuda':
        # transformers' generate() reads every step's logits on the host anyway; the same point checks the error word
        # of the workspaces, so that a kernel's bounded wait that ran out raises instead of yielding wrong tokens
        # (GreedyDecoder.decode does the same for this package's own decoder)
        def _check(module, args, output):
            if not torch.cuda.is_current_stream_capturing():
                _lib.check_exchange_errors()
        model.register_forward_hook(_check)
    return model


def autotune_warmup(model) -> None:
    """Kept for interface compatibility (src/gptq_triton/__init__.py:96-114): the HIP kernels
    choose their launch shape from (M, N, K) directly, so there is no cache to warm."""
    for _ in quant_linear.autotune_warmup(model):
        pass
    for _ in fused_mlp.autotune_warmup(model):
        pass


def save_quant(model, checkpoint: str, wbits: int, groupsize: int, safetensors: bool = True) -> None:
    """Write an UNFUSED quantised model (fresh from make_quant + pack_linear) in the
    reference's checkpoint layout (quantize.py:62-79)."""
    ckpt = Path(checkpoint)
    ckpt.mkdir(parents=True, exist_ok=True)
    state = {k: v.detach().cpu().contiguous() for k, v in model.state_dict().items()}
    if safetensors:
        from safetensors.torch import save_file
        save_file(state, str(ckpt / 'model.safetensors'))
    else:
        torch.save(state, ckpt / 'model.pt')
    json.dump({'wbits': wbits, 'groupsize': groupsize}, open(ckpt / 'quant_config.json', 'w'))
    cfg = model.config
    json.dump({k: getattr(cfg, k) for k in ("hidden_size", "num_attention_heads", "max_position_embeddings",
                                             "rope_theta", "intermediate_size", "num_hidden_layers", "vocab_size",
                                             "rms_norm_eps")} | {"model_type": "llama"},
              open(ckpt / 'config.json', 'w'))
