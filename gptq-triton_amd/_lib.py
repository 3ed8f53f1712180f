"""ctypes binding of csrc/libgptq4.so (the C ABI declared in include/gptq4.h; tuning and test hooks in
include/gptq4_experimental.h).

The HIP library is the only compute path: if it is missing, load() raises, and every
operator that needs it raises with it.  There is no CPU fallback.
"""
from __future__ import annotations

import ctypes
from ctypes import POINTER, Structure, c_char_p, c_float, c_int, c_size_t, c_uint, c_void_p
from pathlib import Path

import torch

LIB_PATH = Path(__file__).resolve().parent / "csrc" / "libgptq4.so"
ABI_VERSION = 3
WS_COUNTER_BYTES = 524288            # arrival counters
WS_HEAD_BYTES = WS_COUNTER_BYTES + (16 << 20)  # GPTQ4_WS_HEAD_BYTES: counters + marked partial sums, zero between calls
WS_ERROR_WORD = 1                     # GPTQ4_WS_ERROR_WORD
STATIC_SCRATCH_BYTES = WS_HEAD_BYTES + (8 << 20)  # GPTQ4_STATIC_SCRATCH_BYTES: what gptq4_matmul_static holds per GPU
OP_MATMUL, OP_MLP_GATEUP, OP_QKV_ROTARY, OP_DECODE_ATTENTION = 0, 1, 2, 3
OP_WITH_PERM = 0x100  # or-ed to a matmul selector in gptq4_workspace_bytes: the call passes `perm`

IN_ROWS, IN_NORM_ROWS, IN_PREV, IN_NORM_PREV = 0, 1, 2, 3     # gptq4_phase_t.input
OUT_NONE, OUT_ROWS, OUT_ROPE = 0, 1, 2                        # gptq4_phase_t.output
CHAIN_MAX_PHASES, CHAIN_MAX_M, CHAIN_ERROR_OFFSET = 8, 4, 4


class Phase(Structure):
    """gptq4_phase_t of include/gptq4.h: one projection of a chained decode launch."""
    _fields_ = [(n, c_void_p) for n in ("qweight", "qzeros", "scales", "up_qweight", "up_qzeros", "up_scales", "perm",
                                        "x", "delta", "norm_weight", "sum_out", "y", "bias", "position_ids",
                                        "cos_table", "sin_table", "q", "k", "v")] + \
               [(n, c_int) for n in ("K", "N", "groupsize", "input", "output")] + [("eps", c_float)] + \
               [(n, c_int) for n in ("H", "max_pos", "kv_capacity", "kv_offset")]


# every symbol include/gptq4.h declares: (restype, argtypes)
SIGNATURES = {
    "gptq4_abi_version": (c_int, []),
    "gptq4_strerror": (c_char_p, [c_int]),
    "gptq4_workspace_bytes": (c_size_t, [c_int, c_int, c_int, c_int]),
    "gptq4_dequant": (c_int, [c_void_p] * 5 + [c_int, c_int, c_int, c_void_p]),
    "gptq4_actorder_sort_rows": (c_int, [c_void_p] * 3 + [c_int, c_int, c_void_p]),
    "gptq4_matmul": (c_int, [c_void_p] * 7 + [c_int] * 4 + [c_void_p, c_size_t, c_void_p]),
    "gptq4_matmul_static": (c_int, [c_void_p] * 6 + [c_int] * 4 + [c_void_p]),
    "gptq4_lm_head_argmax": (c_int, [c_void_p] * 3 + [c_int] * 3 + [c_void_p, c_size_t, c_void_p]),
    "gptq4_prefill_attention": (c_int, [c_void_p] * 4 + [c_int] * 6 + [c_float, c_void_p]),
    "gptq4_static_status": (c_int, [c_void_p]),
    "gptq4_static_reset": (c_int, [c_void_p]),
    "gptq4_mlp_gateup": (c_int, [c_void_p] * 9 + [c_int] * 4 + [c_void_p, c_size_t, c_void_p]),
    "gptq4_rope_table": (c_int, [c_void_p, c_void_p, c_int, c_int, c_float, c_void_p]),
    "gptq4_qkv_rotary": (c_int, [c_void_p] * 8 + [c_int] + [c_void_p] * 3 + [c_int] * 8 + [c_void_p, c_size_t, c_void_p]),
    "gptq4_norm_qkv_rotary": (c_int, [c_void_p] * 3 + [c_float] + [c_void_p] * 8 + [c_int] + [c_void_p] * 3 + [c_int] * 8
                              + [c_void_p, c_size_t, c_void_p]),
    "gptq4_norm_mlp_gateup": (c_int, [c_void_p] * 3 + [c_float] + [c_void_p] * 9 + [c_int] * 4 + [c_void_p, c_size_t, c_void_p]),
    "gptq4_rmsnorm": (c_int, [c_void_p] * 4 + [c_int, c_int, c_float, c_void_p]),
    "gptq4_add_rmsnorm": (c_int, [c_void_p] * 6 + [c_int, c_int, c_float, c_void_p]),
    "gptq4_decode_attention": (c_int, [c_void_p] * 6 + [c_int] * 4 + [c_float, c_void_p, c_size_t, c_void_p]),
    "gptq4_stream_rows": (c_int, [c_int, c_int, c_int, c_int]),
    "gptq4_stream_pack": (c_int, [c_void_p] * 5 + [c_int, c_int, c_int, c_void_p]),
    "gptq4_stream_unpack": (c_int, [c_void_p] * 5 + [c_int, c_int, c_int, c_void_p]),
    "gptq4_stream_dequant": (c_int, [c_void_p] * 3 + [c_int, c_int, c_int, c_void_p]),
    "gptq4_stream_matmul": (c_int, [c_void_p] * 6 + [c_int] * 4 + [c_void_p, c_size_t, c_void_p]),
    "gptq4_stream_mlp_gateup": (c_int, [c_void_p] * 3 + [c_float] + [c_void_p] * 7 + [c_int] * 4 + [c_void_p, c_size_t, c_void_p]),
    "gptq4_stream_qkv_rotary": (c_int, [c_void_p] * 3 + [c_float] + [c_void_p] * 7 + [c_int] + [c_void_p] * 3 + [c_int] * 8
                                + [c_void_p, c_size_t, c_void_p]),
    "gptq4_set_stream_tuning": (None, [c_int, c_int]),
    "gptq4_stream_probe": (c_int, [c_int] + [c_void_p] * 6 + [c_int] * 4 + [c_void_p, c_size_t, c_void_p]),
    "gptq4_chain_workspace_bytes": (c_size_t, [POINTER(Phase), c_int, c_int]),
    "gptq4_decode_chain": (c_int, [POINTER(Phase), c_int, c_int, c_void_p, c_size_t, c_void_p]),
    "gptq4_set_chain_tuning": (None, [c_int, c_int, c_uint, c_int]),
    "gptq4_set_tuning": (None, [c_int, c_int, c_int]),
    "gptq4_set_gemm_tuning": (None, [c_int, c_int]),
    "gptq4_set_midm_tuning": (None, [c_int, c_int, c_int]),
    "gptq4_set_gemv_tuning": (None, [c_int, c_int, c_int, c_int]),
    "gptq4_set_exchange_spin_limit": (None, [ctypes.c_uint]),
    "gptq4_column_parts": (c_int, [c_int, c_int, c_int, c_int, POINTER(c_int), POINTER(c_int)]),
}


class LibraryMissing(RuntimeError):
    pass


_lib = None


def load() -> ctypes.CDLL:
    """Open the in-tree shared object and bind every entry point."""
    global _lib
    if _lib is not None:
        return _lib
    if not LIB_PATH.exists():
        raise LibraryMissing(
            f"{LIB_PATH} is not built; run `python -c 'import __graft_entry__ as g; g.build()'` "
            "or `python gptq-triton_amd/build.py` (needs hipcc)")
    lib = ctypes.CDLL(str(LIB_PATH))
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    got = lib.gptq4_abi_version()
    if got != ABI_VERSION:
        raise LibraryMissing(f"{LIB_PATH} has ABI version {got}, expected {ABI_VERSION}; rebuild it")
    _lib = lib
    return lib


class Gptq4Error(RuntimeError):
    def __init__(self, code: int, where: str):
        self.code = code
        msg = load().gptq4_strerror(code).decode()
        super().__init__(f"{where}: {msg} (code {code})")


def check(code: int, where: str) -> None:
    if code != 0:
        raise Gptq4Error(code, where)


def op_for(op: int, perm) -> int:
    """Selector for gptq4_workspace_bytes: calls that pass `perm` need room for the gathered rows."""
    return op | OP_WITH_PERM if perm is not None else op


def ptr(t: torch.Tensor | None):
    return None if t is None else t.data_ptr()


# (the raw handle without building a torch.cuda.Stream object around it: this is asked twice per launch)
_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def current_stream(device: torch.device):
    if _raw_stream is not None:
        return _raw_stream(device.index if device.index is not None else torch.cuda.current_device())
    return torch.cuda.current_stream(device).cuda_stream


# One workspace per (device, stream): arrival counters and the marked partial sums of the small-M kernels (the
# head, WS_HEAD_BYTES), then plain split-K partial sums (+ the gathered rows of an act-order call).  The head
# must start zeroed; the kernels restore it to zero.
# A workspace that has to grow is replaced by one at least twice as large; the old one is kept
# alive, because captured graphs may still launch kernels that point into it.
_workspaces: dict = {}
_outgrown: list = []
_WS_BYTES = WS_HEAD_BYTES + 16 * 16 * 2 * 32768 * 4  # splitk 16, M 16, 2 matrices, 32768 columns


def workspace(device: torch.device, need: int):
    key = (device.index if device.index is not None else torch.cuda.current_device(), current_stream(device))
    ws = _workspaces.get(key)
    if ws is None or ws.numel() < need:
        if ws is not None:
            _outgrown.append(ws)
        ws = torch.zeros(max(need, _WS_BYTES, 2 * ws.numel() if ws is not None else 0), dtype=torch.uint8, device=device)
        _workspaces[key] = ws
    return ws


def exchange_errors() -> list:
    """(device, stream) keys of the workspaces whose error word is set: a kernel's bounded wait for another
    workgroup's partial sums ran out there, and the results of that call are not valid.  Synchronises."""
    bad = []
    for key, ws in list(_workspaces.items()) + [(None, w) for w in _outgrown]:
        if int(ws[4 * WS_ERROR_WORD:4 * WS_ERROR_WORD + 4].view(torch.int32).item()) != 0:
            bad.append(key)
    return bad


def check_exchange_errors() -> None:
    bad = exchange_errors()
    if bad:
        raise RuntimeError(f"a small-M kernel gave up waiting for partial sums on workspace(s) {bad}: results computed on them "
                           "since the last check are not valid; call reset_workspaces() before reusing them")


def reset_workspaces() -> None:
    """Zero every workspace (after an exchange error, which leaves marked values and the error word behind)."""
    torch.cuda.synchronize()
    for ws in list(_workspaces.values()) + _outgrown:
        ws.zero_()
    torch.cuda.synchronize()


def require_cuda(t: torch.Tensor, name: str) -> None:
    if not t.is_cuda:
        raise RuntimeError(f"{name} must live on the GPU: the HIP library is the only compute path "
                           f"(got device {t.device})")
