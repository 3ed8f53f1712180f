"""MI355X-native 4-bit GPTQ inference hot path.

Same module API as the reference package (src/gptq_triton/__init__.py:10-13):
QuantLinear / make_quant / triton_matmul4, QuantLlamaMLP / make_fused_mlp /
triton_llama_mlp_4, QuantLlamaAttention / make_quant_attn, load_quant,
autotune_warmup - computed by hand-written gfx950 kernels behind a C ABI.
"""
from . import fused_mlp, quant_linear
from .fused_attention import (LlamaConfigLite, QuantLlamaAttention, RotaryTable, make_quant_attn, qkv_rotary, qkv_rotary_stream)
from .fused_mlp import QuantLlamaMLP, llama_mlp_4, llama_mlp_4_stream, make_fused_mlp, triton_llama_mlp_4
from .quant_linear import (QuantLinear, dequantize, make_quant, matmul4, matmul4_stream, prepare_act_order, set_layout, stream_pack,
                           stream_unpack, triton_matmul4)
from .decoder_ops import add_rms_norm, decode_attention, rms_norm
from .llama import GreedyDecoder, LlamaForCausalLM, config_from_json
from .loader import autotune_warmup, load_quant, save_quant
from .pack import pack_linear, quantize_rtn

__all__ = [
    "QuantLinear", "make_quant", "matmul4", "triton_matmul4", "dequantize", "prepare_act_order",
    "QuantLlamaMLP", "make_fused_mlp", "llama_mlp_4", "triton_llama_mlp_4",
    "QuantLlamaAttention", "make_quant_attn", "qkv_rotary", "RotaryTable", "LlamaConfigLite",
    "load_quant", "save_quant", "autotune_warmup", "LlamaForCausalLM", "config_from_json", "pack_linear", "quantize_rtn",
    "GreedyDecoder", "rms_norm", "add_rms_norm", "decode_attention",
    "set_layout", "stream_pack", "stream_unpack", "matmul4_stream", "llama_mlp_4_stream", "qkv_rotary_stream",
]
