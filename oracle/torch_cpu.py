"""The CPU baseline that is timed beside the GPU numbers: dequantise with shifts and
masks, then a float32 matmul, with torch on the host cores.  TEST INFRASTRUCTURE ONLY;
bench.py's cpu_baseline leg and the tests are the only callers.

Same arithmetic as gptq_oracle (quant_linear.py:177-188,211-212 decode; README.md:93
formula) but float32 accumulation inside torch.matmul, which is what
"PyTorch CPU dequantize-then-fp32 matmul" means.
"""
from __future__ import annotations

import torch

_SHIFTS = torch.arange(0, 32, 4, dtype=torch.int32)


def dequant_fp16(qweight: torch.Tensor, qzeros: torch.Tensor, scales: torch.Tensor, groupsize: int,
                 g_idx: torch.Tensor | None = None) -> torch.Tensor:
    rows, n = qweight.shape
    k = rows * 8
    if groupsize == -1:
        groupsize = k
    q = ((qweight[:, None, :] >> _SHIFTS[None, :, None]) & 0xF).reshape(k, n)
    z = ((qzeros[:, :, None] >> _SHIFTS[None, None, :]) & 0xF).reshape(qzeros.shape[0], n)
    g = g_idx.long() if g_idx is not None else torch.arange(k) // groupsize
    d = (q - (z[g] + 1)).float()
    return (d * scales[g].float()).half()


def quant_matmul(x: torch.Tensor, qweight, qzeros, scales, groupsize, bias=None, g_idx=None) -> torch.Tensor:
    w = dequant_fp16(qweight, qzeros, scales, groupsize, g_idx).float()
    y = x.reshape(-1, x.shape[-1]).float() @ w
    if bias is not None:
        y = y + bias.float()
    return y.reshape(x.shape[:-1] + (w.shape[1],))


def mlp(x, gate, up, down, groupsize) -> torch.Tensor:
    """down(silu(gate(x)) * up(x)) with the fp16 intermediate (fused_mlp.py:78-79,222-233)."""
    g = quant_matmul(x, *gate, groupsize)
    u = quant_matmul(x, *up, groupsize)
    h = (torch.nn.functional.silu(g) * u).half()
    return quant_matmul(h, *down, groupsize)
