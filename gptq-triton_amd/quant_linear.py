"""4-bit weight-only linear layer on the HIP kernels.

Mirrors the reference's operator interface for this path (src/gptq_triton/quant_linear.py):
`QuantLinear` (:49-77), `make_quant` (:13-32), the functional `triton_matmul4`
(:228-283; kept as an alias of `matmul4`).  Same buffer names, shapes, dtypes and the
same host-side argument errors; the compute is `gptq4_matmul` of the C ABI.

Extension the reference does not have: an optional `g_idx` buffer (act-order).  Rows are
re-laid-out once, at first use, so each group's rows are contiguous (see
`prepare_act_order`); the checkpoint tensors themselves are never modified.
"""
from __future__ import annotations

import math
from typing import Optional

import torch
import torch.nn as nn

from . import _lib


def _check_matmul_args(a: torch.Tensor, qweight: torch.Tensor, groupsize: int):
    # the reference's host-side contract (quant_linear.py:244-257)
    assert a.shape[-1] == qweight.shape[0] * 8, "A must be a multiple of 8 in the last dimension"
    assert a.is_contiguous(), "A must be contiguous"
    k = a.shape[-1]
    n = qweight.shape[1]
    assert k % 128 == 0, "K must be a multiple of 16, 32, 64, and 128"
    assert n % 256 == 0, "N must be a multiple of 16, 32, 64, 128, and 256"
    assert groupsize % 128 == 0, "groupsize must be a multiple of 32, 64, and 128"
    return k, n


def _check_device_tensors(a, *tensors):
    _lib.require_cuda(a, "activations")
    if a.dtype != torch.float16:
        raise TypeError(f"activations must be float16, got {a.dtype}")
    for t in tensors:
        if t is not None and t.device != a.device:
            raise RuntimeError(f"tensor on {t.device} but activations on {a.device}")
        if t is not None and not t.is_contiguous():
            raise RuntimeError("quantised tensors must be contiguous")


def matmul4(groupsize: int, a: torch.Tensor, qweight: torch.Tensor, scales: torch.Tensor,
            qzeros: torch.Tensor, bias: Optional[torch.Tensor] = None,
            perm: Optional[torch.Tensor] = None) -> torch.Tensor:
    """C = A x dequant(qweight, qzeros, scales) + bias.

    A (..., K) fp16 contiguous; qweight (K//8, N) int32; scales (G, N) fp16; qzeros
    (G, N//8) int32; bias (N) fp16.  Returns (..., N) fp16.  `groupsize` is the number
    of input features per group (K when there is one group).  `perm` is the row
    permutation from `prepare_act_order` (qweight must then be the sorted copy).
    """
    k, n = _check_matmul_args(a, qweight, groupsize)
    _check_device_tensors(a, qweight, scales, qzeros, bias, perm)
    lib = _lib.load()
    x = a.view(-1, k)
    m = x.shape[0]
    c = torch.empty((m, n), device=a.device, dtype=torch.float16)
    if m == 0:
        return c.view(a.shape[:-1] + (n,))
    need = lib.gptq4_workspace_bytes(_lib.op_for(_lib.OP_MATMUL, perm), m, k, n)
    ws = _lib.workspace(a.device, need)
    rc = lib.gptq4_matmul(x.data_ptr(), qweight.data_ptr(), qzeros.data_ptr(), scales.data_ptr(),
                          _lib.ptr(perm), _lib.ptr(bias), c.data_ptr(), m, k, n, groupsize,
                          ws.data_ptr(), ws.numel(), _lib.current_stream(a.device))
    _lib.check(rc, "gptq4_matmul")
    return c.view(a.shape[:-1] + (n,))


# the reference's name for the same functional
triton_matmul4 = matmul4


def dequantize(qweight: torch.Tensor, qzeros: torch.Tensor, scales: torch.Tensor, groupsize: int,
               g_idx: Optional[torch.Tensor] = None) -> torch.Tensor:
    """fp16 [K, N] weight, bit-exact to fp16(float(q - (z + 1)) * float(s))."""
    _lib.require_cuda(qweight, "qweight")
    lib = _lib.load()
    k, n = qweight.shape[0] * 8, qweight.shape[1]
    out = torch.empty((k, n), device=qweight.device, dtype=torch.float16)
    rc = lib.gptq4_dequant(qweight.data_ptr(), qzeros.data_ptr(), scales.data_ptr(), _lib.ptr(g_idx),
                           out.data_ptr(), k, n, groupsize, _lib.current_stream(qweight.device))
    _lib.check(rc, "gptq4_dequant")
    return out


def tensor_key(*tensors):
    """Cache key of derived copies: storage address AND in-place version of every source tensor, so that
    load_state_dict / copy_ into an existing buffer invalidates what was derived from the old contents."""
    return tuple(None if t is None else (t.data_ptr(), t._version, t.device) for t in tensors)


def inverse_permutation(perm: torch.Tensor) -> torch.Tensor:
    """inv with inv[perm[j]] = j: where a producer must store feature f (at inv[f]) so that its output is in the
    order x[:, perm] an act-order projection reads."""
    inv = torch.empty_like(perm)
    inv[perm.long()] = torch.arange(perm.numel(), device=perm.device, dtype=perm.dtype)
    return inv


def _nibble_rows(qweight: torch.Tensor) -> torch.Tensor:
    """[K/8, N] packed words -> [K, N] nibbles (int64), plain torch."""
    shifts = torch.arange(0, 32, 4, device=qweight.device, dtype=torch.int64).view(1, 8, 1)
    return (((qweight.to(torch.int64) & 0xFFFFFFFF).unsqueeze(1) >> shifts) & 0xF).reshape(-1, qweight.shape[1])


def _pack_rows(nibbles: torch.Tensor) -> torch.Tensor:
    """[K, N] nibbles -> [K/8, N] packed int32 words, plain torch."""
    shifts = torch.arange(0, 32, 4, device=nibbles.device, dtype=torch.int64).view(1, 8, 1)
    packed = (nibbles.reshape(-1, 8, nibbles.shape[1]) << shifts).sum(1)
    return torch.where(packed >= 2 ** 31, packed - 2 ** 32, packed).to(torch.int32).contiguous()


def sort_rows(qweight: torch.Tensor, perm: torch.Tensor) -> torch.Tensor:
    """Packed weight whose nibble row j is row perm[j] of `qweight` (perm int32 [K]).  A format conversion, not part
    of the compute path: on the GPU one launch of the library, off it (a model moved to the CPU to be saved) plain
    torch indexing with the same result."""
    if not qweight.is_cuda:
        return _pack_rows(_nibble_rows(qweight).index_select(0, perm.to(device=qweight.device, dtype=torch.int64)))
    out = torch.empty_like(qweight)
    rc = _lib.load().gptq4_actorder_sort_rows(qweight.data_ptr(), perm.data_ptr(), out.data_ptr(), qweight.shape[0] * 8,
                                              qweight.shape[1], _lib.current_stream(qweight.device))
    _lib.check(rc, "gptq4_actorder_sort_rows")
    return out


# ---- streaming-order layout (the decode kernel for up to STREAM_ROWS rows reads it) ------------------------------------
# Per strip of 16 output columns and unit of 128 input rows one contiguous 1 KiB block: lane l = 16 * r + c of a wave
# owns words 4 * l .. 4 * l + 3 of the block, the packed words of the 8-row blocks 4 * r + j (j = 0..3) of the unit, column c
# of the strip; blocks are ordered [strip][unit].  `meta` has one int32 per (strip, group, column): fp16 scale bits |
# stored zero << 16.


def stream_rows(op: int, k: int, n: int, groupsize: int) -> int:
    """Most rows the streaming-order kernels take for this operator and shape (0: the shape is not supported)."""
    return int(_lib.load().gptq4_stream_rows(op, k, n, groupsize))


def stream_workspace_bytes(op: int, m: int, k: int, n: int, with_perm: bool) -> int:
    """Workspace a streaming-order call needs: the zeroed head; for more than four rows of an act-order projection room for
    the gathered rows; above 16 rows what the tiled kernel asks for (it reads the same words)."""
    if m > 16:
        return int(_lib.load().gptq4_workspace_bytes(op | (_lib.OP_WITH_PERM if with_perm else 0), m, k, n))
    return _lib.WS_HEAD_BYTES + (2 * m * k if with_perm and m > 4 else 0)


def _stream_source_index(k: int, n: int, device) -> torch.Tensor:
    """For every word o of the streaming order, its index kb * N + n in the checkpoint order (int64 [K/8 * N])."""
    nb = k // 128
    o = torch.arange((k // 8) * n, device=device, dtype=torch.int64)
    j, lane, blk = o & 3, (o >> 2) & 63, o >> 8
    strip, unit = blk // nb, blk % nb
    return (unit * 16 + 4 * (lane >> 4) + j) * n + strip * 16 + (lane & 15)


def stream_pack(qweight: torch.Tensor, qzeros: Optional[torch.Tensor] = None, scales: Optional[torch.Tensor] = None,
                groupsize: int = -1):
    """(sweight, smeta) of a checkpoint-order projection; smeta is None when qzeros / scales are not given.  sweight
    has qweight's shape and dtype (it is a permutation of its words)."""
    k, n = qweight.shape[0] * 8, qweight.shape[1]
    if not qweight.is_cuda:
        sw = qweight.reshape(-1).index_select(0, _stream_source_index(k, n, qweight.device)).view_as(qweight).contiguous()
        if scales is None:
            return sw, None
        g = scales.shape[0]
        z = ((qzeros.to(torch.int64) & 0xFFFFFFFF).unsqueeze(-1) >> torch.arange(0, 32, 4, dtype=torch.int64)) & 0xF  # [G, N/8, 8]
        word = (scales.view(torch.int16).to(torch.int64) & 0xFFFF) | (z.reshape(g, n) << 16)                          # [G, N]
        return sw, word.view(g, n // 16, 16).transpose(0, 1).reshape(-1).to(torch.int32).contiguous()
    sw = torch.empty_like(qweight)
    gs = k if groupsize == -1 else groupsize
    meta = None if scales is None else torch.empty((k // gs) * n, dtype=torch.int32, device=qweight.device)
    rc = _lib.load().gptq4_stream_pack(qweight.data_ptr(), _lib.ptr(qzeros) if meta is not None else None,
                                       _lib.ptr(scales) if meta is not None else None, sw.data_ptr(), _lib.ptr(meta), k, n, gs,
                                       _lib.current_stream(qweight.device))
    _lib.check(rc, "gptq4_stream_pack")
    return sw, meta


def stream_unpack(sweight: torch.Tensor) -> torch.Tensor:
    """The packed weight in checkpoint order from its streaming-order form (the exact inverse of stream_pack)."""
    k, n = sweight.shape[0] * 8, sweight.shape[1]
    if not sweight.is_cuda:
        out = torch.empty_like(sweight).reshape(-1)
        out[_stream_source_index(k, n, sweight.device)] = sweight.reshape(-1)
        return out.view_as(sweight)
    out = torch.empty_like(sweight)
    rc = _lib.load().gptq4_stream_unpack(sweight.data_ptr(), None, out.data_ptr(), None, None, k, n, -1,
                                         _lib.current_stream(sweight.device))
    _lib.check(rc, "gptq4_stream_unpack")
    return out


def matmul4_stream(groupsize: int, a: torch.Tensor, sweight: torch.Tensor, smeta: torch.Tensor,
                   bias: Optional[torch.Tensor] = None, perm: Optional[torch.Tensor] = None) -> torch.Tensor:
    """matmul4 on a projection in streaming order (stream_pack): A (..., K) fp16 with at most stream_rows() rows."""
    k, n = _check_matmul_args(a, sweight, groupsize)
    _check_device_tensors(a, sweight, smeta, bias, perm)
    lib = _lib.load()
    x = a.view(-1, k)
    m = x.shape[0]
    c = torch.empty((m, n), device=a.device, dtype=torch.float16)
    if m == 0:
        return c.view(a.shape[:-1] + (n,))
    ws = _lib.workspace(a.device, stream_workspace_bytes(_lib.OP_MATMUL, m, k, n, perm is not None))
    rc = lib.gptq4_stream_matmul(x.data_ptr(), sweight.data_ptr(), smeta.data_ptr(), _lib.ptr(perm), _lib.ptr(bias), c.data_ptr(),
                                 m, k, n, groupsize, ws.data_ptr(), ws.numel(), _lib.current_stream(a.device))
    _lib.check(rc, "gptq4_stream_matmul")
    return c.view(a.shape[:-1] + (n,))


def prepare_act_order(qweight: torch.Tensor, g_idx: torch.Tensor, groupsize: int):
    """Load-time re-layout for act-order checkpoints.

    Returns (qweight_sorted, perm): perm = stable argsort of g_idx, qweight_sorted's
    nibble row j is qweight's row perm[j].  Sorted row j then belongs to group
    j // groupsize, which requires every group to own exactly `groupsize` rows (true
    for g_idx made by permuting arange(K) // groupsize).
    """
    _lib.require_cuda(qweight, "qweight")
    k, n = qweight.shape[0] * 8, qweight.shape[1]
    gs = k if groupsize == -1 else groupsize
    g = g_idx.to(torch.int64)
    counts = torch.bincount(g, minlength=math.ceil(k / gs))
    if g.numel() != k or bool((counts != gs).any()):
        raise NotImplementedError("act-order g_idx must assign exactly `groupsize` rows to every group")
    perm = torch.argsort(g, stable=True).to(torch.int32).contiguous()
    return sort_rows(qweight, perm), perm


class QuantLinear(nn.Module):
    """Drop-in for the reference module (quant_linear.py:49-77): same constructor, buffer
    names and shapes.  `act_order=True` additionally registers `g_idx` int32[K]."""

    def __init__(self, bits: int, groupsize: int, infeatures: int, outfeatures: int, bias: bool,
                 act_order: bool = False):
        super().__init__()
        if bits not in [4]:
            raise NotImplementedError("Only 4 bits are supported.")
        groupsize = infeatures if groupsize == -1 else groupsize
        self.infeatures = infeatures
        self.outfeatures = outfeatures
        self.bits = bits
        self.groupsize = groupsize
        features_per_int = 32 // bits
        assert outfeatures % features_per_int == 0, "outfeatures must be a multiple of features_per_int"
        groups = math.ceil(infeatures / groupsize)
        self.register_buffer('qweight', torch.empty((infeatures // features_per_int, outfeatures), dtype=torch.int32))
        self.register_buffer('qzeros', torch.empty((groups, outfeatures // features_per_int), dtype=torch.int32))
        self.register_buffer('scales', torch.empty((groups, outfeatures), dtype=torch.float16))
        if bias:
            self.register_buffer('bias', torch.empty(outfeatures, dtype=torch.float16))
        else:
            self.register_parameter('bias', None)
        if act_order:
            self.register_buffer('g_idx', (torch.arange(infeatures) // groupsize).to(torch.int32))
        else:
            self.g_idx = None
        self._sorted = None  # (key, qweight_sorted, perm), built at first use
        # compact(): `qweight` holds the row-sorted layout and this the permutation that made it
        self.register_buffer('_compact_perm', None, persistent=False)
        # to_stream(): `qweight` holds the streaming-order words (of the row-sorted layout for act-order) and this the
        # {scale, zero} words that go with them; up to _stream_rows rows go to the kernel that reads them
        self.register_buffer('_stream_meta', None, persistent=False)
        self._stream_rows = 0

    def compact(self) -> None:
        """Act-order, on the GPU: keep ONE copy of the packed weight, the row-sorted one the kernels read, in the
        `qweight` buffer (otherwise the sorted copy lives beside the checkpoint tensor).  state_dict() and
        dequantize() still give the checkpoint layout (rows put back on the way out); load_state_dict() brings the
        module back to the checkpoint layout.  Code that reads or writes `.qweight` directly should use
        checkpoint_qweight() / load_state_dict() on a compacted module."""
        if self.g_idx is None or self._compact_perm is not None or self._stream_meta is not None or not self.qweight.is_cuda:
            return
        qs, perm = self._act_order()
        self.qweight = qs
        self._compact_perm = perm
        self._sorted = None

    def to_stream(self) -> bool:
        """On the GPU: keep the packed weight in streaming order - still ONE copy, in the `qweight` buffer - which is
        what the decode kernels for up to `_stream_rows` rows read (an act-order module is compacted first); calls
        with more than 16 rows go to the tiled kernel, which reads the same words.  state_dict(), dequantize() and
        checkpoint_qweight() still give the checkpoint layout (converted on the way out);
        load_state_dict() and to_checkpoint() bring the module back to it.  Returns whether the module now is in
        streaming order (shapes the kernel does not take stay as they are)."""
        if self._stream_meta is not None:
            return True
        if not self.qweight.is_cuda:
            return False
        rows = stream_rows(_lib.OP_MATMUL, self.infeatures, self.outfeatures, self.groupsize)
        if rows == 0:
            return False
        self.compact()
        sw, meta = stream_pack(self.qweight, self.qzeros, self.scales, self.groupsize)
        self.qweight = sw
        self._stream_meta = meta
        self._stream_rows = rows
        self._sorted = None
        return True

    def to_checkpoint(self) -> None:
        """Undo to_stream() (the row order of a compacted act-order module stays sorted: see compact())."""
        if self._stream_meta is not None:
            self.qweight = stream_unpack(self.qweight)
            self._stream_meta = None
            self._stream_rows = 0

    def _kernel_order_qweight(self) -> torch.Tensor:
        """The packed weight in the checkpoint's word layout, rows as the kernels read them."""
        return stream_unpack(self.qweight) if self._stream_meta is not None else self.qweight

    def checkpoint_qweight(self) -> torch.Tensor:
        """The packed weight in the checkpoint's layout and row order."""
        q = self._kernel_order_qweight()
        if self._compact_perm is None:
            return q
        return sort_rows(q, inverse_permutation(self._compact_perm))

    def _save_to_state_dict(self, destination, prefix, keep_vars):
        super()._save_to_state_dict(destination, prefix, keep_vars)
        if self._compact_perm is not None or self._stream_meta is not None:
            destination[prefix + 'qweight'] = self.checkpoint_qweight()

    def _load_from_state_dict(self, state_dict, prefix, *args, **kwargs):
        if self._compact_perm is not None or self._stream_meta is not None:
            self.qweight = self.checkpoint_qweight()
            self._compact_perm = None
            self._stream_meta = None
            self._stream_rows = 0
        super()._load_from_state_dict(state_dict, prefix, *args, **kwargs)

    def _act_order(self):
        key = tensor_key(self.qweight, self.g_idx)
        if self._sorted is None or self._sorted[0] != key:
            qs, perm = prepare_act_order(self.qweight, self.g_idx, self.groupsize)
            self._sorted = (key, qs, perm)
        return self._sorted[1], self._sorted[2]

    def kernel_weights(self):
        """(qweight, perm) as the kernels for the checkpoint order consume them (a module in streaming order unpacks its
        words into a new tensor for this)."""
        if self.g_idx is None:
            return self._kernel_order_qweight(), None
        if self._compact_perm is not None:
            return self._kernel_order_qweight(), self._compact_perm
        return self._act_order()

    def row_permutation(self):
        """perm of kernel_weights() alone (None without act-order)."""
        if self.g_idx is None:
            return None
        return self._compact_perm if self._compact_perm is not None else self._act_order()[1]

    def stream_weights(self, rows: int = 1):
        """(sweight, smeta, perm) if the module is in streaming order, else None (any number of rows: up to `_stream_rows`
        the decode kernels read these words, above that the tiled kernel does)."""
        if self._stream_meta is None or self._stream_rows < rows <= 16:
            return None
        return self.qweight, self._stream_meta, self._compact_perm

    def multiply(self, x: torch.Tensor, ordered: bool = False) -> torch.Tensor:
        """forward(x); ordered: x already is in the order of the sorted rows (act-order), no gather needed."""
        rows = x.numel() // max(self.infeatures, 1)
        sw = self.stream_weights(rows)
        if sw is not None:
            return matmul4_stream(self.groupsize, x, sw[0], sw[1], self.bias, None if ordered else sw[2])
        qweight, perm = self.kernel_weights()
        return matmul4(self.groupsize, x, qweight, self.scales, self.qzeros, self.bias, None if ordered else perm)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return self.multiply(x)

    def dequantize(self) -> torch.Tensor:
        return dequantize(self.checkpoint_qweight(), self.qzeros, self.scales, self.groupsize, self.g_idx)


def make_quant(model: nn.Module, bits: int, groupsize: int, act_order: bool = False):
    """Swap every nn.Linear for a QuantLinear, except the module named exactly
    'lm_head' (quant_linear.py:13-32)."""
    for name, m in list(model.named_modules()):
        if not isinstance(m, nn.Linear) or name == 'lm_head':
            continue
        parent_name, _, child = name.rpartition('.')
        parent = model.get_submodule(parent_name) if parent_name else model
        setattr(parent, child, QuantLinear(bits, groupsize, m.in_features, m.out_features,
                                           m.bias is not None, act_order=act_order))


def autotune_warmup(model):
    """The reference tunes Triton configs per shape here (quant_linear.py:35-46).  The HIP
    kernels pick their launch shape statically, so there is nothing to tune: yields no
    warm-up work and keeps the call site valid."""
    return iter(())


def set_layout(model: nn.Module, layout: str) -> None:
    """'stream': every quantised module of a model on the GPU keeps its packed weights in streaming order (what the
    decode kernel for a handful of rows reads; QuantLinear.to_stream).  'checkpoint': back to the checkpoint's word
    layout.  Either way there is one copy of the weights and state_dict() gives the checkpoint layout."""
    if layout not in ('stream', 'checkpoint'):
        raise ValueError("layout must be 'stream' or 'checkpoint'")
    from .fused_mlp import QuantLlamaMLP
    for m in model.modules():
        if isinstance(m, (QuantLinear, QuantLlamaMLP)):
            m.to_stream() if layout == 'stream' else m.to_checkpoint()


def compact_act_order(model: nn.Module) -> None:
    """compact() every act-order module of a model that is on the GPU: one copy of each packed weight instead of the
    checkpoint tensor plus the layout the kernels read (see QuantLinear.compact)."""
    from .fused_mlp import QuantLlamaMLP
    for m in model.modules():
        if isinstance(m, (QuantLinear, QuantLlamaMLP)):
            m.compact()
