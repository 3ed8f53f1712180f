"""Checkpoint-format packer: float weights + (scale, zero) -> qweight / qzeros / scales in
the exact bit layout the kernels decode.

Mirrors `pack_linear` of the reference (quantize.py:236-291): weights [out, in],
scales / zeros [out, groups]; integer weight = round((w + zero*scale) / scale);
eight 4-bit values per int32 along K for qweight and along N for qzeros; the stored zero
is the true zero minus one.  `quantize_rtn` is the published round-to-nearest min/max
quantiser (the GPTQ paper's baseline, what the reference's `dumbquant` applies,
quantize.py:294-329): per output channel and group, scale = (max - min) / 15 with the
range widened to include 0, zero = round(-min / scale).
CPU-side, load-time code; not on the inference path.  The bit layout is pinned by round trips
through the unpackers; the quantiser's scales, zero points and rounding are pinned by vectors written from
the reference's `Quantizer.find_params` / `quantize` (gptq.py:174-178,205-286; tests/golden/rtn_vectors.npz).
"""
from __future__ import annotations

import torch

from .quant_linear import QuantLinear


@torch.no_grad()
def quantize_rtn(weight: torch.Tensor, groupsize: int = -1, bits: int = 4, packable: bool = True):
    """weight [out, in] -> (dequantised weight [out, in], scale [out, G], zero [out, G]).

    packable=False is the reference's formula as it stands (gptq.py:205-286): a group without a negative weight
    gets zero point 0, which the checkpoint format cannot hold - it stores zero - 1 in four bits
    (quantize.py:276), and the reference's packer then spills into the neighbouring nibbles.  packable=True
    (default) gives such a group the range [-max/14, max] instead: zero point 1, scale max/14, the largest
    weight still on the grid; every other group is quantised exactly as by the reference."""
    w = weight.detach().float().cpu()
    out_f, in_f = w.shape
    gs = in_f if groupsize == -1 else groupsize
    maxq = 2 ** bits - 1
    groups = w.reshape(out_f, in_f // gs, gs)
    wmin = torch.minimum(groups.amin(-1), torch.zeros(()))
    wmax = torch.maximum(groups.amax(-1), torch.zeros(()))
    flat = (wmin == 0) & (wmax == 0)
    wmin = torch.where(flat, torch.full_like(wmin, -1.0), wmin)
    wmax = torch.where(flat, torch.full_like(wmax, 1.0), wmax)
    scale = (wmax - wmin) / maxq
    zero = torch.round(-wmin / scale)
    if packable:
        low = zero < 1
        wmin = torch.where(low, -wmax / (maxq - 1), wmin)
        scale = torch.where(low, (wmax - wmin) / maxq, scale)
        zero = torch.where(low, torch.ones_like(zero), zero)
    q = torch.clamp(torch.round(groups / scale[..., None]) + zero[..., None], 0, maxq)
    deq = (scale[..., None] * (q - zero[..., None])).reshape(out_f, in_f)
    return deq, scale, zero


@torch.no_grad()
def pack_linear(quant: QuantLinear, weights: torch.Tensor, scales: torch.Tensor, zeros: torch.Tensor,
                bias: torch.Tensor | None = None) -> None:
    """Fill `quant`'s buffers.  weights [out, in] (already on the quantisation grid or not:
    they are rounded to it), scales / zeros [out, G] with zeros the TRUE zero points."""
    w = weights.detach().float().cpu()
    s = scales.detach().float().cpu().t().contiguous()   # [G, out]
    z = zeros.detach().float().cpu().t().contiguous()
    k, n = quant.infeatures, quant.outfeatures
    gidx = torch.arange(k) // quant.groupsize
    # integer weights, [K, N]
    q = torch.round((w.t() + (z * s)[gidx]) / s[gidx]).to(torch.int64)
    if int(q.min()) < 0 or int(q.max()) > 15:
        raise ValueError("weights fall outside the 4-bit grid of the given scales / zeros")
    zs = (z - 1).to(torch.int64)
    if int(zs.min()) < 0 or int(zs.max()) > 15:
        raise ValueError("zero points must lie in [1, 16] (they are stored minus one in 4 bits)")
    shifts = (4 * torch.arange(8, dtype=torch.int64))
    qw = (q.reshape(k // 8, 8, n) << shifts[None, :, None]).sum(1)
    qz = (zs.reshape(zs.shape[0], n // 8, 8) << shifts[None, None, :]).sum(2)
    to_i32 = lambda t: torch.where(t >= 2 ** 31, t - 2 ** 32, t).to(torch.int32)
    quant.qweight = to_i32(qw).contiguous()
    quant.qzeros = to_i32(qz).contiguous()
    quant.scales = s.to(torch.float16).contiguous()
    if quant.bias is not None and bias is not None:
        quant.bias = bias.detach().clone().to(torch.float16)
