"""Fused LLaMA MLP on the HIP kernels: h = silu(x @ Wgate) * (x @ Wup) in one launch
(`gptq4_mlp_gateup`), then down_proj as an ordinary QuantLinear.

Mirrors src/gptq_triton/fused_mlp.py of the reference: `QuantLlamaMLP` (:52-79, note
the constructor order gate, down, up), `make_fused_mlp` (:13-27) and the functional
`triton_llama_mlp_4` (:241-302; kept as an alias of `llama_mlp_4`).
"""
from __future__ import annotations

from typing import Optional

import torch
import torch.nn as nn

from . import _lib
from .quant_linear import (QuantLinear, _check_device_tensors, _check_matmul_args, matmul4, stream_pack, stream_rows, stream_workspace_bytes,
                           stream_unpack, tensor_key)


def llama_mlp_4(groupsize: int, a: torch.Tensor,
                gate_qweight: torch.Tensor, gate_scales: torch.Tensor, gate_qzeros: torch.Tensor,
                up_qweight: torch.Tensor, up_scales: torch.Tensor, up_qzeros: torch.Tensor,
                perm: Optional[torch.Tensor] = None) -> torch.Tensor:
    """silu(gate(a)) * up(a).  A (..., K) fp16; *_qweight (K//8, N) int32; *_scales (G, N)
    fp16; *_qzeros (G, N//8) int32.  Returns (..., N) fp16.  SiLU and the product are
    taken on the fp32 accumulators and rounded once."""
    assert (gate_qweight.shape == up_qweight.shape and gate_scales.shape == up_scales.shape
            and gate_qzeros.shape == up_qzeros.shape), "All weights must have the same shape"
    k, n = _check_matmul_args(a, gate_qweight, groupsize)
    _check_device_tensors(a, gate_qweight, gate_scales, gate_qzeros, up_qweight, up_scales, up_qzeros, perm)
    lib = _lib.load()
    x = a.view(-1, k)
    m = x.shape[0]
    c = torch.empty((m, n), device=a.device, dtype=torch.float16)
    if m == 0:
        return c.view(a.shape[:-1] + (n,))
    need = lib.gptq4_workspace_bytes(_lib.op_for(_lib.OP_MLP_GATEUP, perm), m, k, n)
    ws = _lib.workspace(a.device, need)
    rc = lib.gptq4_mlp_gateup(x.data_ptr(), gate_qweight.data_ptr(), gate_qzeros.data_ptr(), gate_scales.data_ptr(),
                              up_qweight.data_ptr(), up_qzeros.data_ptr(), up_scales.data_ptr(), _lib.ptr(perm),
                              c.data_ptr(), m, k, n, groupsize, ws.data_ptr(), ws.numel(),
                              _lib.current_stream(a.device))
    _lib.check(rc, "gptq4_mlp_gateup")
    return c.view(a.shape[:-1] + (n,))


triton_llama_mlp_4 = llama_mlp_4


def norm_llama_mlp_4(groupsize: int, h: torch.Tensor, delta: Optional[torch.Tensor], norm_weight: torch.Tensor, eps: float,
                     gate_qweight: torch.Tensor, gate_scales: torch.Tensor, gate_qzeros: torch.Tensor,
                     up_qweight: torch.Tensor, up_scales: torch.Tensor, up_qzeros: torch.Tensor,
                     perm: Optional[torch.Tensor] = None):
    """(s, silu(gate(xn)) * up(xn)) with s = h + delta (h when delta is None) and xn = RMSNorm(s) * norm_weight,
    in ONE launch: the kernel normalises its own input.  Same bits as add_rms_norm followed by llama_mlp_4.
    Decode-sized inputs only (decoder_ops.norm_fusable)."""
    from .decoder_ops import check_norm_args, norm_fusable
    assert (gate_qweight.shape == up_qweight.shape and gate_scales.shape == up_scales.shape
            and gate_qzeros.shape == up_qzeros.shape), "All weights must have the same shape"
    k, n = _check_matmul_args(h, gate_qweight, groupsize)
    _check_device_tensors(h, gate_qweight, gate_scales, gate_qzeros, up_qweight, up_scales, up_qzeros, perm)
    h2, d2, s = check_norm_args(h, delta, norm_weight)
    m = h2.shape[0]
    if not norm_fusable(m, k):
        raise ValueError(f"{m} rows of {k} values are outside what the fused norm takes; run add_rms_norm and llama_mlp_4")
    lib = _lib.load()
    c = torch.empty((m, n), device=h.device, dtype=torch.float16)
    ws = _lib.workspace(h.device, lib.gptq4_workspace_bytes(_lib.OP_MLP_GATEUP, m, k, n))
    rc = lib.gptq4_norm_mlp_gateup(h2.data_ptr(), _lib.ptr(d2), norm_weight.data_ptr(), float(eps), _lib.ptr(s),
                                   gate_qweight.data_ptr(), gate_qzeros.data_ptr(), gate_scales.data_ptr(),
                                   up_qweight.data_ptr(), up_qzeros.data_ptr(), up_scales.data_ptr(), _lib.ptr(perm),
                                   c.data_ptr(), m, k, n, groupsize, ws.data_ptr(), ws.numel(), _lib.current_stream(h.device))
    _lib.check(rc, "gptq4_norm_mlp_gateup")
    return (h if s is None else s.view(h.shape)), c.view(h.shape[:-1] + (n,))


def llama_mlp_4_stream(groupsize: int, a: torch.Tensor, gate_sweight: torch.Tensor, gate_smeta: torch.Tensor,
                       up_sweight: torch.Tensor, up_smeta: torch.Tensor, perm: Optional[torch.Tensor] = None, norm=None):
    """llama_mlp_4 on projections in streaming order (quant_linear.stream_pack), for up to stream_rows() rows.
    norm = (delta or None, norm_weight, eps): `a` is the residual stream h and the kernel multiplies with
    RMSNorm(h + delta) * norm_weight; returns (h + delta, result) then."""
    assert gate_sweight.shape == up_sweight.shape and gate_smeta.shape == up_smeta.shape, "All weights must have the same shape"
    k, n = _check_matmul_args(a, gate_sweight, groupsize)
    _check_device_tensors(a, gate_sweight, gate_smeta, up_sweight, up_smeta, perm)
    lib = _lib.load()
    delta_p = nw_p = sum_p = None
    eps = 0.0
    x, s = a.view(-1, k), None
    if norm is not None:
        from .decoder_ops import check_norm_args
        delta, norm_weight, eps = norm
        x, d2, s = check_norm_args(a, delta, norm_weight)
        delta_p, nw_p, sum_p = _lib.ptr(d2), norm_weight.data_ptr(), _lib.ptr(s)
    m = x.shape[0]
    c = torch.empty((m, n), device=a.device, dtype=torch.float16)
    if m:
        ws = _lib.workspace(a.device, stream_workspace_bytes(_lib.OP_MLP_GATEUP, m, k, n, perm is not None))
        rc = lib.gptq4_stream_mlp_gateup(x.data_ptr(), delta_p, nw_p, float(eps), sum_p, gate_sweight.data_ptr(), gate_smeta.data_ptr(),
                                         up_sweight.data_ptr(), up_smeta.data_ptr(), _lib.ptr(perm), c.data_ptr(), m, k, n, groupsize,
                                         ws.data_ptr(), ws.numel(), _lib.current_stream(a.device))
        _lib.check(rc, "gptq4_stream_mlp_gateup")
    out = c.view(a.shape[:-1] + (n,))
    if norm is None:
        return out
    return (a if s is None else s.view(a.shape)), out


def _move_zero_columns(qzeros: torch.Tensor, cols: torch.Tensor) -> torch.Tensor:
    """qzeros [G, N/8] (eight 4-bit stored zeros per word, column 8c+t in bits [4t, 4t+4)) with its
    columns gathered: column j of the result = column cols[j] of the input."""
    shifts = torch.arange(0, 32, 4, device=qzeros.device, dtype=torch.int64)
    z = ((qzeros.to(torch.int64) & 0xFFFFFFFF).unsqueeze(-1) >> shifts) & 0xF   # [G, N/8, 8]
    z = z.reshape(qzeros.shape[0], -1).index_select(1, cols).reshape(qzeros.shape[0], -1, 8)
    packed = (z << shifts).sum(-1)
    packed = torch.where(packed >= 2 ** 31, packed - 2 ** 32, packed)
    return packed.to(torch.int32).contiguous()


class QuantLlamaMLP(nn.Module):
    """forward(x) = down_proj(silu(gate(x)) * up(x)).  Holds the six gate/up tensors as its
    own buffers under the reference's names and keeps down_proj as a submodule
    (fused_mlp.py:52-79)."""

    def __init__(self, gate_proj: QuantLinear, down_proj: QuantLinear, up_proj: QuantLinear):
        super().__init__()
        assert gate_proj.groupsize == up_proj.groupsize
        self.register_buffer('gate_proj_qweight', gate_proj.checkpoint_qweight())
        self.register_buffer('gate_proj_scales', gate_proj.scales)
        self.register_buffer('gate_proj_qzeros', gate_proj.qzeros)
        self.register_buffer('up_proj_qweight', up_proj.checkpoint_qweight())
        self.register_buffer('up_proj_scales', up_proj.scales)
        self.register_buffer('up_proj_qzeros', up_proj.qzeros)
        self.groupsize = gate_proj.groupsize
        self.infeatures = gate_proj.infeatures
        self.outfeatures = down_proj.outfeatures
        self.down_proj = down_proj
        # act-order: the gate and up rows must be sorted by ONE permutation because the
        # kernel streams x once for both (they share their input, hence their g_idx)
        g_gate, g_up = getattr(gate_proj, 'g_idx', None), getattr(up_proj, 'g_idx', None)
        if (g_gate is None) != (g_up is None) or (g_gate is not None and not torch.equal(g_gate.cpu(), g_up.cpu())):
            raise NotImplementedError("gate_proj and up_proj must share one g_idx to be fused")
        if g_gate is not None:
            self.register_buffer('g_idx', g_gate)
        else:
            self.g_idx = None
        self._sorted = None
        self._chained = None
        self._input_order = None
        # compact(): the six gate / up buffers hold the layout forward() multiplies with; these say how it was made
        self._is_compact = False
        self.register_buffer('_compact_rows', None, persistent=False)   # row permutation (act-order input), or None
        self.register_buffer('_compact_cols', None, persistent=False)   # column order (act-order down_proj), or None
        # to_stream(): the two qweight buffers hold streaming-order words (of the layout above) and these the {scale, zero}
        # words that go with them
        self.register_buffer('_gate_meta', None, persistent=False)
        self.register_buffer('_up_meta', None, persistent=False)
        self._stream_rows = 0

    _SIX = ('gate_proj_qweight', 'gate_proj_scales', 'gate_proj_qzeros', 'up_proj_qweight', 'up_proj_scales', 'up_proj_qzeros')

    def compact(self) -> None:
        """Act-order, on the GPU: keep ONE copy of the gate and up tensors, in the layout forward() reads (rows sorted
        by group, columns in the order of an act-order down_proj's rows), in the module's own buffers - otherwise that
        layout lives beside the checkpoint tensors.  state_dict() still gives the checkpoint layout (rows and columns
        put back on the way out) and load_state_dict() brings the module back to it."""
        if self._is_compact or self._gate_meta is not None or not self.gate_proj_qweight.is_cuda:
            return
        self.down_proj.compact()
        w, perm, _ = self._chained_weights()
        down_perm = self.down_proj.row_permutation()
        if perm is None and down_perm is None:
            return
        for name, t in zip(self._SIX, w):
            setattr(self, name, t)
        self._compact_rows = perm
        self._compact_cols = None if down_perm is None else down_perm.long()
        self._is_compact = True
        self._sorted = self._chained = None

    def to_stream(self) -> bool:
        """On the GPU: gate, up (and down_proj) keep their packed weights in streaming order, which the decode kernel
        for up to `_stream_rows` rows reads - still one copy (see QuantLinear.to_stream; an act-order block is
        compacted first).  Returns whether gate and up now are in streaming order."""
        if self._gate_meta is not None:
            return True
        if not self.gate_proj_qweight.is_cuda:
            return False
        self.compact()  # (act-order: rows sorted, columns in down_proj's order, while down_proj still is in the checkpoint's word layout)
        self.down_proj.to_stream()
        rows = stream_rows(_lib.OP_MLP_GATEUP, self.infeatures, self.gate_proj_qweight.shape[1], self.groupsize)
        if rows == 0 or ((self.g_idx is not None or self.down_proj.g_idx is not None) and not self._is_compact):
            return False
        self.gate_proj_qweight, self._gate_meta = stream_pack(self.gate_proj_qweight, self.gate_proj_qzeros, self.gate_proj_scales, self.groupsize)
        self.up_proj_qweight, self._up_meta = stream_pack(self.up_proj_qweight, self.up_proj_qzeros, self.up_proj_scales, self.groupsize)
        self._stream_rows = rows
        self._sorted = self._chained = None
        return True

    def to_checkpoint(self) -> None:
        """Undo to_stream() (a compacted act-order block stays compacted)."""
        self.down_proj.to_checkpoint()
        if self._gate_meta is not None:
            self.gate_proj_qweight = stream_unpack(self.gate_proj_qweight)
            self.up_proj_qweight = stream_unpack(self.up_proj_qweight)
            self._gate_meta = self._up_meta = None
            self._stream_rows = 0

    def _six(self) -> tuple:
        """The six gate / up tensors in the checkpoint's word layout (rows and columns as the kernels read them)."""
        out = [getattr(self, name) for name in self._SIX]
        if self._gate_meta is not None:
            out[0], out[3] = stream_unpack(out[0]), stream_unpack(out[3])
        return tuple(out)

    def checkpoint_tensors(self) -> dict:
        """The six gate / up tensors in the checkpoint's layout, by buffer name."""
        out = dict(zip(self._SIX, self._six()))
        if not self._is_compact:
            return out
        from .quant_linear import inverse_permutation, sort_rows
        if self._compact_cols is not None:
            inv = inverse_permutation(self._compact_cols)
            for name in self._SIX:
                out[name] = _move_zero_columns(out[name], inv) if name.endswith('qzeros') else out[name].index_select(1, inv).contiguous()
        if self._compact_rows is not None:
            back = inverse_permutation(self._compact_rows)
            for name in ('gate_proj_qweight', 'up_proj_qweight'):
                out[name] = sort_rows(out[name], back)
        return out

    def _save_to_state_dict(self, destination, prefix, keep_vars):
        super()._save_to_state_dict(destination, prefix, keep_vars)
        if self._is_compact or self._gate_meta is not None:
            for name, t in self.checkpoint_tensors().items():
                destination[prefix + name] = t

    def _load_from_state_dict(self, state_dict, prefix, *args, **kwargs):
        if self._is_compact or self._gate_meta is not None:
            for name, t in self.checkpoint_tensors().items():
                setattr(self, name, t)
            self._is_compact = False
            self._compact_rows = self._compact_cols = None
            self._gate_meta = self._up_meta = None
            self._stream_rows = 0
        super()._load_from_state_dict(state_dict, prefix, *args, **kwargs)

    def _kernel_weights(self):
        if self._is_compact:
            raise RuntimeError("a compacted module multiplies through _chained_weights()")
        if self.g_idx is None:
            return self.gate_proj_qweight, self.up_proj_qweight, None
        key = tensor_key(self.gate_proj_qweight, self.up_proj_qweight, self.g_idx)
        if self._sorted is None or self._sorted[0] != key:
            from .quant_linear import prepare_act_order
            gq, perm = prepare_act_order(self.gate_proj_qweight, self.g_idx, self.groupsize)
            uq, _ = prepare_act_order(self.up_proj_qweight, self.g_idx, self.groupsize)
            self._sorted = (key, gq, uq, perm)
        return self._sorted[1], self._sorted[2], self._sorted[3]

    def gate_up(self, x: torch.Tensor) -> torch.Tensor:
        if self._is_compact:
            mid = llama_mlp_4(self.groupsize, x, *self._six(), self._compact_rows)
            if self._compact_cols is None:
                return mid
            from .quant_linear import inverse_permutation
            return mid.index_select(-1, inverse_permutation(self._compact_cols))
        if self._gate_meta is not None:
            return llama_mlp_4(self.groupsize, x, *self._six(), None)
        gq, uq, perm = self._kernel_weights()
        return llama_mlp_4(self.groupsize, x, gq, self.gate_proj_scales, self.gate_proj_qzeros,
                           uq, self.up_proj_scales, self.up_proj_qzeros, perm)

    def _chained_weights(self):
        """The tensors forward() multiplies with: (gate/up set, input permutation, down_proj's sorted qweight).

        With an act-order down_proj the OUTPUT columns of gate and up are laid out once in the order of
        down_proj's sorted rows (column j of the copies = column perm_down[j] of the originals: a
        column only moves, its values do not change).  The intermediate then comes out of the gate/up
        launch already in the order down_proj's kernel reads, and down_proj runs without a gather."""
        down_q, down_perm = self.down_proj.kernel_weights()
        if self._is_compact or self._gate_meta is not None:
            return self._six(), self._compact_rows, down_q
        if down_perm is None:
            gq, uq, perm = self._kernel_weights()
            return (gq, self.gate_proj_scales, self.gate_proj_qzeros, uq, self.up_proj_scales, self.up_proj_qzeros), perm, down_q
        key = tensor_key(self.gate_proj_qweight, self.up_proj_qweight, self.gate_proj_scales, self.up_proj_scales,
                         self.gate_proj_qzeros, self.up_proj_qzeros, down_perm, self.g_idx)
        if self._chained is None or self._chained[0] != key:
            cols = down_perm.long()
            if self.g_idx is None:
                gq, uq, perm = self.gate_proj_qweight, self.up_proj_qweight, None
            else:
                from .quant_linear import prepare_act_order
                gq, perm = prepare_act_order(self.gate_proj_qweight, self.g_idx, self.groupsize)
                uq, _ = prepare_act_order(self.up_proj_qweight, self.g_idx, self.groupsize)
            tensors = (gq.index_select(1, cols).contiguous(), self.gate_proj_scales.index_select(1, cols).contiguous(),
                       _move_zero_columns(self.gate_proj_qzeros, cols),
                       uq.index_select(1, cols).contiguous(), self.up_proj_scales.index_select(1, cols).contiguous(),
                       _move_zero_columns(self.up_proj_qzeros, cols))
            self._chained = (key, tensors, perm)
            # the row-sorted copies were only a step on the way: beside the checkpoint tensors (which state_dict
            # needs) the module keeps ONE derived copy of gate and up; gate_up() rebuilds the sorted pair if asked
            self._sorted = None
            del gq, uq
        return self._chained[1], self._chained[2], down_q

    def _down(self, mid: torch.Tensor, down_q: torch.Tensor) -> torch.Tensor:
        d = self.down_proj
        return matmul4(d.groupsize, mid, down_q, d.scales, d.qzeros, d.bias, None)

    def input_order(self):
        """Where a producer should store each input feature so that x arrives in the order gate and up read it
        (int32 [infeatures], the inverse of their shared permutation; None without act-order):
        rms_norm / add_rms_norm(out_index=...) write in that order and forward(x, ordered=True) runs
        without a gather."""
        perm = self._compact_rows if (self._is_compact or self._gate_meta is not None) else self._chained_weights()[1]
        if perm is None:
            return None
        if self._input_order is None or self._input_order[0] != tensor_key(perm):
            from .quant_linear import inverse_permutation
            self._input_order = (tensor_key(perm), inverse_permutation(perm))
        return self._input_order[1]

    def _stream_ready(self, x: torch.Tensor) -> bool:
        # (any number of rows: the decode kernels up to _stream_rows, the tiled kernel above 16)
        rows = x.numel() // max(self.infeatures, 1)
        return self._gate_meta is not None and not (self._stream_rows < rows <= 16)

    def forward(self, x: torch.Tensor, ordered: bool = False) -> torch.Tensor:
        if self._stream_ready(x):
            mid = llama_mlp_4_stream(self.groupsize, x, self.gate_proj_qweight, self._gate_meta, self.up_proj_qweight, self._up_meta,
                                     None if ordered else self._compact_rows)
            return self.down_proj.multiply(mid, ordered=True)  # the columns of gate and up are laid out in the order down_proj reads
        w, perm, down_q = self._chained_weights()
        return self._down(llama_mlp_4(self.groupsize, x, *w, None if ordered else perm), down_q)

    def norm_fusable(self, rows: int) -> bool:
        """Whether forward_normed is the faster way for this many rows."""
        from .decoder_ops import norm_fusion_pays
        return norm_fusion_pays(rows, self.infeatures)

    def forward_normed(self, h: torch.Tensor, delta: Optional[torch.Tensor], norm_weight: torch.Tensor, eps: float):
        """(h + delta, forward(RMSNorm(h + delta))): the residual add and the norm run inside the gate/up launch."""
        from .decoder_ops import NORM_MAX_ROWS
        if self._stream_ready(h) and h.numel() // self.infeatures <= NORM_MAX_ROWS:
            s, mid = llama_mlp_4_stream(self.groupsize, h, self.gate_proj_qweight, self._gate_meta, self.up_proj_qweight, self._up_meta,
                                        self._compact_rows, norm=(delta, norm_weight, eps))
            return s, self.down_proj.multiply(mid, ordered=True)
        w, perm, down_q = self._chained_weights()
        s, mid = norm_llama_mlp_4(self.groupsize, h, delta, norm_weight, eps, *w, perm)
        return s, self._down(mid, down_q)


def _is_llama_mlp(m: nn.Module) -> bool:
    """An MLP block with three quantised projections named as in LLaMA."""
    if isinstance(m, QuantLlamaMLP):
        return False
    return all(isinstance(getattr(m, n, None), QuantLinear) for n in ('gate_proj', 'down_proj', 'up_proj'))


def make_fused_mlp(m: nn.Module, parent_name: str = ''):
    """Replace every LLaMA MLP block under `m` by a QuantLlamaMLP; returns `m` itself, or
    its replacement when `m` is such a block (fused_mlp.py:13-27)."""
    if _is_llama_mlp(m):
        return QuantLlamaMLP(m.gate_proj, m.down_proj, m.up_proj)
    for name, child in list(m.named_children()):
        new = make_fused_mlp(child, parent_name=f"{parent_name}.{name}")
        if new is not child:
            setattr(m, name, new)
    return m


def autotune_warmup(model):
    """Nothing to tune (see quant_linear.autotune_warmup); reference: fused_mlp.py:30-49."""
    return iter(())
