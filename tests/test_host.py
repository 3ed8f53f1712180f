"""Host-side checks that need no GPU: the C-ABI library loads and exports every symbol
include/gptq4.h declares, argument errors are raised before any launch, and the module
API keeps the reference's names, shapes and error behaviour."""
import ctypes
import os
import re

import numpy as np
import pytest
import torch
import torch.nn as nn

import gptq_triton_amd as G
from gptq_triton_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols(header):
    text = open(os.path.join(ROOT, "include", header)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(gptq4_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    lib = _lib.load()
    stable, experimental = declared_symbols("gptq4.h"), declared_symbols("gptq4_experimental.h")
    assert len(stable) >= 20
    for name in stable + experimental:
        assert hasattr(lib, name), f"{name} declared in include/ but not exported"
    assert set(stable + experimental) == set(_lib.SIGNATURES), "ctypes binding and headers disagree"
    # the stable header carries no tuning, probe or test hook
    assert not [n for n in stable if "_set_" in n or "probe" in n or "chain" in n or "column_parts" in n]
    assert lib.gptq4_abi_version() == 3


def test_error_codes_are_returned_before_any_launch():
    lib = _lib.load()
    fake = 0x1000  # never dereferenced: the host rejects the call first
    ws = 1 << 20
    # NULL pointer
    assert lib.gptq4_matmul(None, fake, fake, fake, None, None, fake, 1, 4096, 4096, -1, fake, ws, None) == -1
    # K not a multiple of 128 / N not a multiple of 256 / M < 1
    assert lib.gptq4_matmul(fake, fake, fake, fake, None, None, fake, 1, 4000, 4096, -1, fake, ws, None) == -2
    assert lib.gptq4_matmul(fake, fake, fake, fake, None, None, fake, 1, 4096, 4100, -1, fake, ws, None) == -2
    assert lib.gptq4_matmul(fake, fake, fake, fake, None, None, fake, 0, 4096, 4096, -1, fake, ws, None) == -2
    # groupsize must divide K and be a multiple of 128
    assert lib.gptq4_matmul(fake, fake, fake, fake, None, None, fake, 1, 4096, 4096, 96, fake, ws, None) == -3
    assert lib.gptq4_matmul(fake, fake, fake, fake, None, None, fake, 1, 4096, 4096, 384, fake, ws, None) == -3
    # workspace too small for the split-K partial sums
    assert lib.gptq4_matmul(fake, fake, fake, fake, None, None, fake, 1, 4096, 4096, -1, fake, 64, None) == -4
    assert lib.gptq4_matmul(fake, fake, fake, fake, None, None, fake, 1, 4096, 4096, -1, None, 0, None) == -4
    # misaligned pointer
    assert lib.gptq4_matmul(fake + 2, fake, fake, fake, None, None, fake, 1, 4096, 4096, -1, fake, ws, None) == -5
    # rotary: head_dim must be 128, cache must have room
    args = [fake] * 4 + [None] + [fake] * 3
    assert lib.gptq4_qkv_rotary(*args, 2048, fake, fake, fake, 1, 1, 32, 64, 4096, -1, 1, 0, fake, ws, None) == -2
    assert lib.gptq4_qkv_rotary(*args, 2048, fake, fake, fake, 1, 4, 32, 128, 4096, -1, 3, 0, fake, ws, None) == -2
    assert lib.gptq4_mlp_gateup(fake, fake, fake, fake, None, fake, fake, None, fake, 1, 4096, 11008, -1, fake, ws, None) == -1
    # the entry point with its own scratch memory: argument errors first, then its size limit - all before any GPU call
    assert lib.gptq4_matmul_static(None, fake, fake, fake, None, fake, 1, 4096, 4096, -1, None) == -1
    assert lib.gptq4_matmul_static(fake, fake, fake, fake, None, fake, 1, 4096, 4096, 96, None) == -3
    assert lib.gptq4_matmul_static(fake, fake, fake, fake, None, fake, 16, 4096, 32768, -1, None) == -6
    for code in (0, -1, -2, -3, -4, -5, -6):
        assert len(lib.gptq4_strerror(code)) > 0


def test_workspace_query():
    lib = _lib.load()
    base = _lib.WS_HEAD_BYTES
    assert lib.gptq4_workspace_bytes(_lib.OP_MATMUL, 4096, 4096, 12288) == base   # enough tiles: no split-K, only the counters
    one = lib.gptq4_workspace_bytes(_lib.OP_MATMUL, 1, 4096, 4096)
    assert one >= base + 16 * 1 * 4096 * 4                    # 16 split-K slots at least; the decode GEMV may want more
    assert lib.gptq4_workspace_bytes(_lib.OP_MLP_GATEUP, 16, 4096, 11008) == base + 16 * 16 * 2 * 11008 * 4
    # mid-M on a narrow layer: 32 tiles of 128x128, split 8 ways, 64 KiB of fp32 per tile and split
    assert lib.gptq4_workspace_bytes(_lib.OP_MATMUL, 128, 4096, 4096) == base + 32 * 8 * 65536
    # a call that will pass `perm` also needs room for its gathered rows (M * K fp16 values) ...
    for op, m, k, n in ((_lib.OP_MATMUL, 4096, 4096, 12288), (_lib.OP_MLP_GATEUP, 16, 4096, 11008), (_lib.OP_QKV_ROTARY, 128, 4096, 12288)):
        assert lib.gptq4_workspace_bytes(op | _lib.OP_WITH_PERM, m, k, n) == lib.gptq4_workspace_bytes(op, m, k, n) + m * k * 2
    # ... unless they pass the staging limit (1 GiB): the tiled kernel gathers such rows itself
    assert lib.gptq4_workspace_bytes(_lib.OP_MATMUL | _lib.OP_WITH_PERM, 32768, 17920, 6656) == base


def test_quant_linear_layout_and_errors():
    q = G.QuantLinear(4, 128, 4096, 11008, bias=False)
    assert q.qweight.shape == (512, 11008) and q.qweight.dtype == torch.int32
    assert q.qzeros.shape == (32, 1376) and q.qzeros.dtype == torch.int32
    assert q.scales.shape == (32, 11008) and q.scales.dtype == torch.float16
    assert q.bias is None and sorted(q.state_dict()) == ["qweight", "qzeros", "scales"]
    assert (q.infeatures, q.outfeatures, q.bits, q.groupsize) == (4096, 11008, 4, 128)
    q = G.QuantLinear(4, -1, 4096, 4096, bias=True)
    assert q.groupsize == 4096 and q.qzeros.shape == (1, 512) and q.scales.shape == (1, 4096)
    assert q.bias.shape == (4096,) and "bias" in q.state_dict()
    assert len(list(q.parameters())) == 0                     # buffers, not parameters
    q = G.QuantLinear(4, 128, 256, 256, bias=False, act_order=True)
    assert q.g_idx.dtype == torch.int32 and (q.g_idx == torch.arange(256) // 128).all()
    with pytest.raises(NotImplementedError, match="Only 4 bits"):
        G.QuantLinear(3, -1, 4096, 4096, bias=False)
    with pytest.raises(AssertionError):
        G.QuantLinear(4, -1, 4096, 4100, bias=False)


def test_functional_argument_errors_come_first():
    qw = torch.zeros((512, 4096), dtype=torch.int32)
    sc = torch.zeros((1, 4096), dtype=torch.float16)
    qz = torch.zeros((1, 512), dtype=torch.int32)
    with pytest.raises(AssertionError):   # K mismatch
        G.triton_matmul4(4096, torch.zeros((1, 4000), dtype=torch.float16), qw, sc, qz)
    with pytest.raises(AssertionError):   # non-contiguous activations
        G.triton_matmul4(4096, torch.zeros((4096, 2), dtype=torch.float16).t(), qw, sc, qz)
    with pytest.raises(AssertionError):   # N not a multiple of 256
        G.triton_matmul4(4096, torch.zeros((1, 4096), dtype=torch.float16), qw[:, :4000].contiguous(), sc, qz)
    with pytest.raises(AssertionError):   # groupsize not a multiple of 128
        G.triton_matmul4(64, torch.zeros((1, 4096), dtype=torch.float16), qw, sc, qz)
    with pytest.raises(AssertionError):   # K not a multiple of 128
        G.triton_matmul4(64, torch.zeros((1, 64), dtype=torch.float16), qw[:8], sc, qz)
    with pytest.raises(AssertionError, match="same shape"):
        G.triton_llama_mlp_4(4096, torch.zeros((1, 4096), dtype=torch.float16), qw, sc, qz, qw[:, :2048], sc, qz)
    # no CPU fallback: host tensors are refused loudly
    with pytest.raises(RuntimeError, match="GPU"):
        G.triton_matmul4(4096, torch.zeros((1, 4096), dtype=torch.float16), qw, sc, qz)


class _Attn(nn.Module):
    def __init__(self, h):
        super().__init__()
        self.config = G.LlamaConfigLite(hidden_size=h, num_attention_heads=h // 128)
        self.q_proj, self.k_proj, self.v_proj, self.o_proj = (nn.Linear(h, h, bias=False) for _ in range(4))


class _MLP(nn.Module):
    def __init__(self, h, i):
        super().__init__()
        self.gate_proj, self.up_proj, self.down_proj = nn.Linear(h, i, bias=False), nn.Linear(h, i, bias=False), nn.Linear(i, h, bias=False)


class _Block(nn.Module):
    def __init__(self, h, i):
        super().__init__()
        self.self_attn, self.mlp = _Attn(h), _MLP(h, i)


class _Model(nn.Module):
    def __init__(self, h=256, i=512):
        super().__init__()
        self.layers = nn.ModuleList([_Block(h, i), _Block(h, i)])
        self.lm_head = nn.Linear(h, 1000, bias=False)


def test_model_surgery_keeps_reference_names():
    model = _Model()
    G.make_quant(model, 4, 128)
    assert isinstance(model.lm_head, nn.Linear)              # the module named 'lm_head' is skipped
    assert isinstance(model.layers[0].self_attn.q_proj, G.QuantLinear)
    keys = set(model.state_dict())
    assert "layers.1.mlp.down_proj.qweight" in keys and "layers.0.self_attn.k_proj.scales" in keys
    # distinguishable content to check the concatenation order q, k, v
    for li in range(2):
        a = model.layers[li].self_attn
        for v, p in enumerate((a.q_proj, a.k_proj, a.v_proj)):
            p.qweight.fill_(v + 1); p.qzeros.fill_(v + 11); p.scales.fill_(v + 21)
    G.make_quant_attn(model)
    attn = model.layers[0].self_attn
    assert isinstance(attn, G.QuantLlamaAttention)
    qkv = attn.qkv_proj
    assert qkv.outfeatures == 768 and qkv.qweight.shape == (32, 768) and qkv.qzeros.shape == (2, 96)
    assert qkv.qweight[0, 0] == 1 and qkv.qweight[0, 256] == 2 and qkv.qweight[0, 512] == 3
    assert qkv.qzeros[0, 31] == 11 and qkv.qzeros[0, 32] == 12 and qkv.scales[1, 767] == 23
    assert (attn.hidden_size, attn.num_heads, attn.head_dim) == (256, 2, 128)
    out = G.make_fused_mlp(model)
    assert out is model
    mlp = model.layers[1].mlp
    assert isinstance(mlp, G.QuantLlamaMLP)
    names = set(dict(mlp.named_buffers(recurse=False)))
    assert names == {"gate_proj_qweight", "gate_proj_scales", "gate_proj_qzeros",
                     "up_proj_qweight", "up_proj_scales", "up_proj_qzeros"}
    assert isinstance(mlp.down_proj, G.QuantLinear)
    assert (mlp.infeatures, mlp.outfeatures, mlp.groupsize) == (256, 256, 128)
    # called on an MLP block itself, make_fused_mlp returns the replacement
    m2 = _MLP(256, 512)
    holder = nn.Module(); holder.m = m2
    G.make_quant(holder, 4, -1)
    assert isinstance(G.make_fused_mlp(holder.m), G.QuantLlamaMLP)


def test_attention_config_error():
    cfg = G.LlamaConfigLite(hidden_size=300, num_attention_heads=7)
    with pytest.raises(ValueError, match="divisible"):
        G.QuantLlamaAttention(cfg, None, None, None)


def test_product_code_never_touches_the_oracle():
    pkg = os.path.join(ROOT, "gptq-triton_amd")
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".h", ".cpp")):
                text = open(os.path.join(dirpath, f)).read()
                assert "oracle" not in text.lower() or f == "never", f"{f} mentions the oracle"


def test_bench_refuses_more_than_one_gpu():
    """Every box has one GPU: `bench.py --gpus N` with N > 1 must say so and exit non-zero
    without touching a device."""
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert r.returncode != 0
    assert "one GPU" in (r.stderr + r.stdout) or "single GPU" in (r.stderr + r.stdout) or "--gpus 1" in (r.stderr + r.stdout)


def test_mid_m_plan_is_declared_and_tunable():
    """The launch-plan hooks exist with the documented arity (no compute is launched)."""
    from gptq_triton_amd import _lib
    lib = _lib.load()
    for args in ((0, 0, 0), (2, 1, 3), (1, 0, 0)):
        lib.gptq4_set_midm_tuning(*args)
    # the workspace query covers whichever kernel the plans pick for a mid-sized call
    assert lib.gptq4_workspace_bytes(_lib.OP_MATMUL, 64, 4096, 4096) >= _lib.WS_HEAD_BYTES
    assert lib.gptq4_workspace_bytes(_lib.OP_QKV_ROTARY, 128, 4096, 12288) >= _lib.WS_HEAD_BYTES


def test_column_parts_plan_without_a_gpu():
    """The plan that cuts a call into two launches over column ranges is host arithmetic (256 CUs assumed where no
    device can be asked): LLaMA-7B gate/up has 86 column tiles, so 6 or 12 row tiles are 4 or 8 tiles more than an
    even number of rounds; 3 row tiles (2 over one round) and 4 (88 over) are cut along K inside one launch instead,
    decode-sized calls are never cut; the tuning hook switches it off."""
    import ctypes
    lib = _lib.load()

    def parts(op, m, k, n):
        begin, cols = (ctypes.c_int * 2)(), (ctypes.c_int * 2)()
        count = lib.gptq4_column_parts(op, m, k, n, begin, cols)
        return [(begin[i], cols[i]) for i in range(count)]

    assert parts(_lib.OP_MLP_GATEUP, 384, 4096, 11008) == [(0, 11008)]                            # 258 tiles: cut along K instead
    assert parts(_lib.OP_MLP_GATEUP, 768, 4096, 11008) == [(0, 85 * 128), (85 * 128, 128)]       # 516 tiles: 512 + 4
    assert parts(_lib.OP_MLP_GATEUP, 1536, 4096, 11008) == [(0, 85 * 128), (85 * 128, 128)]      # 1032: 1024 + 8
    assert parts(_lib.OP_MLP_GATEUP, 512, 4096, 11008) == [(0, 11008)]
    assert parts(_lib.OP_MLP_GATEUP, 1, 4096, 11008) == [(0, 11008)]
    assert parts(_lib.OP_MATMUL, 2048, 4096, 4096) == [(0, 4096)]
    lib.gptq4_set_gemm_tuning(300, 0)
    try:
        assert parts(_lib.OP_MLP_GATEUP, 768, 4096, 11008) == [(0, 11008)]
    finally:
        lib.gptq4_set_gemm_tuning(0, 0)
    assert parts(_lib.OP_QKV_ROTARY, 1408, 4096, 12288) == [(0, 46 * 256), (46 * 256, 2 * 256)]  # 11 x 48 = 528: 512 + 16
    assert parts(_lib.OP_QKV_ROTARY, 768, 4096, 12288) == [(0, 12288)]                            # the mid-M kernel takes it whole


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    """No CPU fallback: with the shared object absent, loading raises and names the build command."""
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", tmp_path / "libgptq4.so")
    with pytest.raises(_lib.LibraryMissing, match="build"):
        _lib.load()
    layer = G.QuantLinear(4, 128, 256, 256, bias=False)
    with pytest.raises((_lib.LibraryMissing, RuntimeError, AssertionError)):
        layer(torch.zeros((1, 256), dtype=torch.float16))


def test_norm_entry_points_check_their_arguments_on_the_host():
    lib = _lib.load()
    fake, ws = 0x1000, 1 << 20

    def gateup(m, k, delta, weight, sums):
        return lib.gptq4_norm_mlp_gateup(fake, delta, weight, 1e-6, sums, fake, fake, fake, fake, fake, fake, None, fake,
                                         m, k, 11008, 128, fake, ws, None)

    assert gateup(1, 4096, fake, None, fake) == -1            # no norm weight
    assert gateup(1, 4096, fake, fake, None) == -1            # a delta but nowhere to put the sums
    assert gateup(5, 4096, fake, fake, 0x2000) == -2          # more rows than the kernels normalise themselves
    assert gateup(1, 8192 + 128, fake, fake, 0x2000) == -2    # rows longer than they keep in registers
    assert gateup(1, 4096, fake, fake, fake) == -2            # sums over the input
    assert gateup(1, 4096, 0x3000, fake, 0x3000) == -2        # sums over the delta
    assert gateup(1, 4096, fake + 2, fake, 0x2000) == -5      # misaligned delta
    args = [fake, None, None, 1e-6, None, fake, fake, fake, None, fake, fake, fake, 2048, fake, fake, fake]
    assert lib.gptq4_norm_qkv_rotary(*args, 1, 1, 32, 128, 4096, -1, 1, 0, fake, ws, None) == -1   # no norm weight
