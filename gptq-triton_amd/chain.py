"""Chained decode launch: several decode-sized quantised projections in ONE persistent launch
(`gptq4_decode_chain` of the C ABI).

The reference launches one Triton kernel per projection (quant_linear.py:264-274, fused_mlp.py:286-297) with the
decoder layer's torch ops between them; here a list of phases - each a QuantLinear or a gate/up pair with what
feeds it (rows in memory, the previous phase's output, optionally through a residual add + RMSNorm) - runs on
one resident grid that streams all their weights as one sequence.
"""
from __future__ import annotations

from typing import Optional, Sequence

import torch

from . import _lib
from ._lib import IN_NORM_PREV, IN_NORM_ROWS, IN_PREV, IN_ROWS, OUT_NONE, OUT_ROPE, OUT_ROWS, Phase

MAX_ROWS = _lib.CHAIN_MAX_M
MAX_PHASES = _lib.CHAIN_MAX_PHASES


def _p(t: Optional[torch.Tensor]):
    return None if t is None else t.data_ptr()


def projection(qweight: torch.Tensor, qzeros: torch.Tensor, scales: torch.Tensor, groupsize: int, *,
               up: Optional[Sequence[torch.Tensor]] = None, input: int = IN_ROWS, x: Optional[torch.Tensor] = None,
               delta: Optional[torch.Tensor] = None, norm_weight: Optional[torch.Tensor] = None, eps: float = 0.0,
               sum_out: Optional[torch.Tensor] = None, output: int = OUT_NONE, y: Optional[torch.Tensor] = None,
               bias: Optional[torch.Tensor] = None, rope: Optional[dict] = None) -> Phase:
    """One phase.  `up` = (qweight, qzeros, scales) of the up matrix makes it a gate/up pair (SiLU*mul).
    rope = dict(position_ids int32 [M], cos, sin float32 [max_pos, 64], q, k, v, heads, kv_offset) for OUT_ROPE."""
    ph = Phase()
    ph.qweight, ph.qzeros, ph.scales = qweight.data_ptr(), qzeros.data_ptr(), scales.data_ptr()
    if up is not None:
        ph.up_qweight, ph.up_qzeros, ph.up_scales = (t.data_ptr() for t in up)
    ph.K, ph.N, ph.groupsize = qweight.shape[0] * 8, qweight.shape[1], groupsize
    ph.input, ph.output, ph.eps = input, output, float(eps)
    ph.x, ph.delta, ph.norm_weight, ph.sum_out, ph.y, ph.bias = _p(x), _p(delta), _p(norm_weight), _p(sum_out), _p(y), _p(bias)
    if rope is not None:
        kc = rope["k"]
        ph.position_ids, ph.cos_table, ph.sin_table = rope["position_ids"].data_ptr(), rope["cos"].data_ptr(), rope["sin"].data_ptr()
        ph.q, ph.k, ph.v = rope["q"].data_ptr(), kc.data_ptr(), rope["v"].data_ptr()
        ph.H, ph.max_pos, ph.kv_capacity, ph.kv_offset = rope["heads"], rope["cos"].shape[0], kc.shape[2], rope.get("kv_offset", 0)
    return ph


# one chain workspace per (device, stream, byte size): it carries state between launches and starts zeroed
_workspaces: dict = {}


def workspace(device: torch.device, nbytes: int) -> torch.Tensor:
    key = (device.index if device.index is not None else torch.cuda.current_device(),
           torch.cuda.current_stream(device).cuda_stream)
    ws = _workspaces.get(key)
    if ws is None or ws.numel() < nbytes:
        ws = torch.zeros(max(nbytes, 1 << 20), dtype=torch.uint8, device=device)  # an outgrown one stays alive in graphs that hold it
        _workspaces[key] = ws
    return ws


def error_word(ws: torch.Tensor) -> int:
    """0, or the code of the launch that gave up on this workspace (synchronises)."""
    return int(ws[_lib.CHAIN_ERROR_OFFSET:_lib.CHAIN_ERROR_OFFSET + 4].view(torch.int32).item())


def decode_chain(phases: Sequence[Phase], rows: int, device: torch.device, ws: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Launch the chain on the current stream; returns the workspace it used."""
    lib = _lib.load()
    arr = (Phase * len(phases))(*phases)
    need = lib.gptq4_chain_workspace_bytes(arr, len(phases), rows)
    if need == 0:
        # let the launch call say why
        _lib.check(lib.gptq4_decode_chain(arr, len(phases), rows, None, 0, _lib.current_stream(device)), "gptq4_decode_chain")
        raise ValueError("gptq4_chain_workspace_bytes rejected the phase list")
    if ws is None:
        ws = workspace(device, need)
    rc = lib.gptq4_decode_chain(arr, len(phases), rows, ws.data_ptr(), ws.numel(), _lib.current_stream(device))
    _lib.check(rc, "gptq4_decode_chain")
    return ws
