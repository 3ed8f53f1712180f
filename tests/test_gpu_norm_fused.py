"""GPU tests of the projections that normalise their own input (gptq4_norm_qkv_rotary,
gptq4_norm_mlp_gateup): the same bits as the residual add + RMSNorm launch followed by the plain
projection, the oracle's values within the stated tolerance, argument errors, and a greedy
decoder whose every token equals the one of the separate-launch path."""
import numpy as np
import pytest
import torch

from conftest import to_dev
from oracle import gptq_oracle as O
from test_gpu_parity import assert_close, gptq

pytestmark = pytest.mark.gpu


@pytest.fixture
def split_k_kernel_only():
    """The one-row gate/up pair normally takes the balanced GEMV, whose summation order differs:
    switch it off so that both sides of a bit-for-bit comparison run the split-K kernel."""
    from gptq_triton_amd import _lib
    lib = _lib.load()
    lib.gptq4_set_gemv_tuning(0, 0, 0, 0)
    yield lib
    lib.gptq4_set_gemv_tuning(1, 0, 0, 0)


@pytest.fixture(params=[1, 2], ids=["gemv_auto", "gemv_everywhere"])
def balanced_gemv(request):
    """The balanced GEMV where it is the default (one-row gate/up pair) and forced on for every call it can take."""
    from gptq_triton_amd import _lib
    lib = _lib.load()
    lib.gptq4_set_gemv_tuning(request.param, 0, 0, 0)
    yield lib
    lib.gptq4_set_gemv_tuning(1, 0, 0, 0)


def residual_inputs(m, hidden, seed):
    rng = np.random.default_rng(seed)
    h = (rng.standard_normal((m, hidden)) * 2).astype(np.float16)
    d = rng.standard_normal((m, hidden)).astype(np.float16)
    w = (1.0 + 0.1 * rng.standard_normal(hidden)).astype(np.float16)
    return h, d, w


@pytest.mark.parametrize("hidden,heads,g", [(1024, 8, 128), (4096, 32, -1)])
@pytest.mark.parametrize("m", [1, 2, 3, 4])
@pytest.mark.parametrize("with_delta", [True, False])
def test_norm_qkv_rotary_equals_two_launches(split_k_kernel_only, hidden, heads, g, m, with_delta):
    G = gptq()
    from gptq_triton_amd.decoder_ops import add_rms_norm, rms_norm
    L = O.make_layer(hidden, 3 * hidden, g, seed=500 + hidden)
    D = to_dev(L)
    gs = hidden if g == -1 else g
    h, d, w = residual_inputs(m, hidden, seed=m + 7)
    hd, dd, wd = (torch.from_numpy(t).cuda() for t in (h, d, w))
    hd, dd = hd.view(m, 1, hidden), dd.view(m, 1, hidden)
    pos = torch.arange(m, dtype=torch.int32, device="cuda").view(m, 1) * 5 + 3
    cos, sin = G.RotaryTable(128, 2048).get(torch.device("cuda"), 2048)
    eps = 1e-6
    if with_delta:
        s_ref, x_ref = add_rms_norm(hd, dd, wd, eps)
    else:
        s_ref, x_ref = hd, rms_norm(hd, wd, eps)
    q0, k0, v0 = G.qkv_rotary(gs, x_ref, D["qweight"], D["scales"], D["qzeros"], pos, cos, sin, heads)
    h_before, d_before = hd.clone(), dd.clone()
    q, k, v, s = G.qkv_rotary(gs, hd, D["qweight"], D["scales"], D["qzeros"], pos, cos, sin, heads,
                              norm=(dd if with_delta else None, wd, eps))
    assert torch.equal(q, q0) and torch.equal(k, k0) and torch.equal(v, v0)
    assert torch.equal(s, s_ref)
    assert torch.equal(hd, h_before) and torch.equal(dd, d_before), "inputs must stay untouched"
    if m == 1 and hidden == 1024:
        # against the oracle end to end
        x_or = O.rmsnorm_ref((h.astype(np.float32) + (d.astype(np.float32) if with_delta else 0)).astype(np.float16), w, eps)
        qr, kr, vr = O.qkv_rotary_ref(x_or.reshape(m, 1, hidden), L["qweight"], L["qzeros"], L["scales"], g,
                                      pos.cpu().numpy(), heads, 128, max_pos=2048)
        assert_close(q.cpu().numpy(), qr, "fused norm + qkv, q")
        assert_close(v.cpu().numpy(), vr, "fused norm + qkv, v")


@pytest.mark.parametrize("hidden,inter,g", [(1024, 2816 - 2816 % 256, 128), (4096, 11008, 128)])
@pytest.mark.parametrize("m", [1, 2, 4])
@pytest.mark.parametrize("with_delta", [True, False])
def test_norm_mlp_gateup_equals_two_launches(split_k_kernel_only, hidden, inter, g, m, with_delta):
    G = gptq()
    from gptq_triton_amd.decoder_ops import add_rms_norm, rms_norm
    from gptq_triton_amd.fused_mlp import norm_llama_mlp_4
    gate, up = O.make_layer(hidden, inter, g, seed=600), O.make_layer(hidden, inter, g, seed=601)
    Dg, Du = to_dev(gate), to_dev(up)
    h, d, w = residual_inputs(m, hidden, seed=m + 17)
    hd, dd, wd = (torch.from_numpy(t).cuda() for t in (h, d, w))
    eps = 1e-5
    if with_delta:
        s_ref, x_ref = add_rms_norm(hd, dd, wd, eps)
    else:
        s_ref, x_ref = hd, rms_norm(hd, wd, eps)
    mid0 = G.llama_mlp_4(g, x_ref, Dg["qweight"], Dg["scales"], Dg["qzeros"], Du["qweight"], Du["scales"], Du["qzeros"])
    s, mid = norm_llama_mlp_4(g, hd, dd if with_delta else None, wd, eps, Dg["qweight"], Dg["scales"], Dg["qzeros"],
                              Du["qweight"], Du["scales"], Du["qzeros"])
    assert torch.equal(mid, mid0) and torch.equal(s, s_ref)
    # twice in a row: the counters and the LDS staging leave nothing behind
    s2, mid2 = norm_llama_mlp_4(g, hd, dd if with_delta else None, wd, eps, Dg["qweight"], Dg["scales"], Dg["qzeros"],
                                Du["qweight"], Du["scales"], Du["qzeros"])
    assert torch.equal(mid2, mid) and torch.equal(s2, s)


@pytest.mark.parametrize("m", [1, 2, 4])
def test_norm_in_the_balanced_gemv_equals_two_launches(balanced_gemv, m):
    """Same comparison through the balanced GEMV's self-normalising variant (gate/up and QKV + rotary)."""
    G = gptq()
    from gptq_triton_amd.decoder_ops import add_rms_norm
    from gptq_triton_amd.fused_mlp import norm_llama_mlp_4
    hidden, inter, heads, g = 4096, 11008, 32, 128
    gate, up = O.make_layer(hidden, inter, g, seed=700), O.make_layer(hidden, inter, g, seed=701)
    qkv = O.make_layer(hidden, 3 * hidden, g, seed=702)
    Dg, Du, Dq = to_dev(gate), to_dev(up), to_dev(qkv)
    h, d, w = residual_inputs(m, hidden, seed=m + 27)
    hd, dd, wd = (torch.from_numpy(t).cuda() for t in (h, d, w))
    eps = 1e-6
    s_ref, x_ref = add_rms_norm(hd, dd, wd, eps)
    mid0 = G.llama_mlp_4(g, x_ref, Dg["qweight"], Dg["scales"], Dg["qzeros"], Du["qweight"], Du["scales"], Du["qzeros"])
    s, mid = norm_llama_mlp_4(g, hd, dd, wd, eps, Dg["qweight"], Dg["scales"], Dg["qzeros"],
                              Du["qweight"], Du["scales"], Du["qzeros"])
    assert torch.equal(mid, mid0) and torch.equal(s, s_ref)
    ref = O.mlp_gateup_ref(x_ref.cpu().numpy(), (gate["qweight"], gate["qzeros"], gate["scales"]),
                           (up["qweight"], up["qzeros"], up["scales"]), g)
    assert_close(mid.cpu().numpy(), ref, f"norm + gate/up M={m}")
    pos = torch.full((m, 1), 2047, dtype=torch.int32, device="cuda")
    cos, sin = G.RotaryTable(128, 2048).get(torch.device("cuda"), 2048)
    q0, k0, v0 = G.qkv_rotary(g, x_ref.view(m, 1, hidden), Dq["qweight"], Dq["scales"], Dq["qzeros"], pos, cos, sin, heads)
    q, k, v, s2 = G.qkv_rotary(g, hd.view(m, 1, hidden), Dq["qweight"], Dq["scales"], Dq["qzeros"], pos, cos, sin, heads,
                               norm=(dd.view(m, 1, hidden), wd, eps))
    assert torch.equal(q, q0) and torch.equal(k, k0) and torch.equal(v, v0) and torch.equal(s2.view(m, hidden), s_ref)
    from gptq_triton_amd import _lib
    ws = _lib.workspace(hd.device, 0)
    torch.cuda.synchronize()
    assert int(ws[:_lib.WS_HEAD_BYTES].view(torch.int32).abs().sum()) == 0


@pytest.mark.parametrize("gemv_mode", [0, 2])
@pytest.mark.parametrize("m", [1, 3])
def test_norm_with_act_order_equals_two_launches(gemv_mode, m):
    """Act-order layers: the kernels gather the permuted activations from the normalised row in LDS."""
    from gptq_triton_amd import _lib
    from gptq_triton_amd.decoder_ops import add_rms_norm
    from test_gpu_baseline_shapes import quant_linear
    G = gptq()
    hidden, inter, g = 1024, 768, 128
    gate = O.make_layer(hidden, inter, g, seed=800, act_order=True)
    up = O.make_layer(hidden, inter, g, seed=801)
    up["g_idx"] = gate["g_idx"]
    down = O.make_layer(inter, hidden, g, seed=802, act_order=True)
    mlp = G.QuantLlamaMLP(quant_linear(gate, hidden, inter, g, True), quant_linear(down, inter, hidden, g, True),
                          quant_linear(up, hidden, inter, g, True)).cuda()
    h, d, w = residual_inputs(m, hidden, seed=m + 37)
    hd, dd, wd = (torch.from_numpy(t).cuda() for t in (h, d, w))
    lib = _lib.load()
    lib.gptq4_set_gemv_tuning(gemv_mode, 0, 0, 0)
    try:
        s_ref, x_ref = add_rms_norm(hd, dd, wd, 1e-6)
        y_ref = mlp(x_ref)
        s, y = mlp.forward_normed(hd, dd, wd, 1e-6)
    finally:
        lib.gptq4_set_gemv_tuning(1, 0, 0, 0)
    assert torch.equal(s, s_ref) and torch.equal(y, y_ref)
    # the same through the rotary epilogue
    heads = hidden // 128
    qkv = O.make_layer(hidden, 3 * hidden, g, seed=803)
    Dq = to_dev(qkv)
    qq, perm = G.prepare_act_order(Dq["qweight"], torch.from_numpy(gate["g_idx"]).cuda(), g)
    cos, sin = G.RotaryTable(128, 2048).get(torch.device("cuda"), 2048)
    pos = torch.full((m, 1), 9, dtype=torch.int32, device="cuda")
    lib.gptq4_set_gemv_tuning(gemv_mode, 0, 0, 0)
    try:
        q0, k0, v0 = G.qkv_rotary(g, x_ref.view(m, 1, hidden), qq, Dq["scales"], Dq["qzeros"], pos, cos, sin, heads, perm=perm)
        q, k, v, s3 = G.qkv_rotary(g, hd.view(m, 1, hidden), qq, Dq["scales"], Dq["qzeros"], pos, cos, sin, heads, perm=perm,
                                   norm=(dd.view(m, 1, hidden), wd, 1e-6))
    finally:
        lib.gptq4_set_gemv_tuning(1, 0, 0, 0)
    assert torch.equal(q, q0) and torch.equal(k, k0) and torch.equal(v, v0) and torch.equal(s3.view(m, hidden), s_ref)
    ref = O.mlp_gateup_ref(x_ref.cpu().numpy(), (gate["qweight"], gate["qzeros"], gate["scales"], gate["g_idx"]),
                           (up["qweight"], up["qzeros"], up["scales"], up["g_idx"]), g)
    assert_close(mlp.gate_up(x_ref).cpu().numpy(), ref, "act-order gate/up on the normalised rows")


# (four rows of 6656 or 8192 values leave the balanced GEMV no room in its 64 KiB of LDS: the self-normalising call
# then runs the split-K kernel whatever the mode, so only mode 0 compares like with like)
@pytest.mark.parametrize("act_order", [False, True])
@pytest.mark.parametrize("hidden,m,gemv_mode", [(5120, 1, 0), (5120, 1, 2), (5120, 3, 0), (5120, 3, 2), (6656, 4, 0), (8192, 4, 0)])
def test_norm_with_rows_longer_than_4096(gemv_mode, act_order, hidden, m):
    """Hidden sizes above 4096: four chunks per thread cover a row (the variants LLaMA-13B / 30B decoders run).
    Four rows of 6656 or 8192 values are the largest calls the entry points accept: 52 and 64 KiB of normalised
    rows in LDS on top of the kernel's 16 KiB reduction buffer."""
    from gptq_triton_amd import _lib
    from gptq_triton_amd.decoder_ops import add_rms_norm
    from gptq_triton_amd.fused_mlp import norm_llama_mlp_4
    G = gptq()
    inter, heads, g = 2816, hidden // 128, 128
    gate = O.make_layer(hidden, inter, g, seed=850, act_order=act_order)
    up = O.make_layer(hidden, inter, g, seed=851)
    qkv = O.make_layer(hidden, 3 * hidden, g, seed=852)
    up["g_idx"] = qkv["g_idx"] = gate["g_idx"]
    Dg, Du, Dq = to_dev(gate), to_dev(up), to_dev(qkv)
    gq, uq, qq, perm = Dg["qweight"], Du["qweight"], Dq["qweight"], None
    if act_order:
        gq, perm = G.prepare_act_order(Dg["qweight"], Dg["g_idx"], g)
        uq, _ = G.prepare_act_order(Du["qweight"], Dg["g_idx"], g)
        qq, _ = G.prepare_act_order(Dq["qweight"], Dg["g_idx"], g)
    h, d, w = residual_inputs(m, hidden, seed=m + 47)
    hd, dd, wd = (torch.from_numpy(t).cuda() for t in (h, d, w))
    pos = torch.full((m, 1), 100, dtype=torch.int32, device="cuda")
    cos, sin = G.RotaryTable(128, 2048).get(torch.device("cuda"), 2048)
    lib = _lib.load()
    lib.gptq4_set_gemv_tuning(gemv_mode, 0, 0, 0)
    try:
        s_ref, x_ref = add_rms_norm(hd, dd, wd, 1e-6)
        mid0 = G.llama_mlp_4(g, x_ref, gq, Dg["scales"], Dg["qzeros"], uq, Du["scales"], Du["qzeros"], perm=perm)
        q0, k0, v0 = G.qkv_rotary(g, x_ref.view(m, 1, hidden), qq, Dq["scales"], Dq["qzeros"], pos, cos, sin, heads, perm=perm)
        s, mid = norm_llama_mlp_4(g, hd, dd, wd, 1e-6, gq, Dg["scales"], Dg["qzeros"], uq, Du["scales"], Du["qzeros"], perm=perm)
        q, k, v, s2 = G.qkv_rotary(g, hd.view(m, 1, hidden), qq, Dq["scales"], Dq["qzeros"], pos, cos, sin, heads, perm=perm,
                                   norm=(dd.view(m, 1, hidden), wd, 1e-6))
    finally:
        lib.gptq4_set_gemv_tuning(1, 0, 0, 0)
    assert torch.equal(s, s_ref) and torch.equal(s2.view(m, hidden), s_ref)
    assert torch.equal(mid, mid0)
    assert torch.equal(q, q0) and torch.equal(k, k0) and torch.equal(v, v0)
    gi = gate["g_idx"]
    ref = O.mlp_gateup_ref(x_ref.cpu().numpy(), (gate["qweight"], gate["qzeros"], gate["scales"], gi),
                           (up["qweight"], up["qzeros"], up["scales"], gi), g)
    assert_close(mid.cpu().numpy(), ref, f"norm + gate/up hidden {hidden} M={m}")


def test_norm_entry_points_reject_what_they_cannot_take():
    from gptq_triton_amd import _lib
    from gptq_triton_amd.fused_mlp import norm_llama_mlp_4
    G = gptq()
    lib = _lib.load()
    hidden, inter, g = 1024, 512, 128
    gate, up = O.make_layer(hidden, inter, g, seed=1), O.make_layer(hidden, inter, g, seed=2)
    Dg, Du = to_dev(gate), to_dev(up)
    w = torch.ones(hidden, dtype=torch.float16, device="cuda")
    with pytest.raises(ValueError):   # 5 rows: the Python layer refuses before the call
        norm_llama_mlp_4(g, torch.zeros((5, hidden), dtype=torch.float16, device="cuda"), None, w, 1e-6,
                         Dg["qweight"], Dg["scales"], Dg["qzeros"], Du["qweight"], Du["scales"], Du["qzeros"])
    x = torch.zeros((2, hidden), dtype=torch.float16, device="cuda")
    d = torch.zeros_like(x)
    out = torch.empty((2, inter), dtype=torch.float16, device="cuda")
    ws = _lib.workspace(x.device, lib.gptq4_workspace_bytes(_lib.OP_MLP_GATEUP, 2, hidden, inter))

    def call(xp, dp, sp, m):
        return lib.gptq4_norm_mlp_gateup(xp, dp, w.data_ptr(), 1e-6, sp, Dg["qweight"].data_ptr(), Dg["qzeros"].data_ptr(),
                                         Dg["scales"].data_ptr(), Du["qweight"].data_ptr(), Du["qzeros"].data_ptr(),
                                         Du["scales"].data_ptr(), None, out.data_ptr(), m, hidden, inter, g, ws.data_ptr(),
                                         ws.numel(), _lib.current_stream(x.device))

    s = torch.empty_like(x)
    assert call(x.data_ptr(), d.data_ptr(), s.data_ptr(), 2) == 0
    assert call(x.data_ptr(), d.data_ptr(), x.data_ptr(), 2) == -2      # sums over the input
    assert call(x.data_ptr(), d.data_ptr(), d.data_ptr(), 2) == -2      # sums over the delta
    assert call(x.data_ptr(), d.data_ptr(), None, 2) == -1              # delta without a place for the sums
    assert call(x.data_ptr(), d.data_ptr(), s.data_ptr(), 5) == -2      # too many rows
    torch.cuda.synchronize()


@pytest.mark.parametrize("bsz,act_order", [(1, False), (3, False), (2, True)])
def test_decoder_with_norm_in_matmul_gives_the_same_tokens(tmp_path, split_k_kernel_only, monkeypatch, bsz, act_order):
    """GreedyDecoder takes the 5-launch layer when it can; its tokens (eager and graph-replayed) equal
    those of the 7-launch layer."""
    import gptq_triton_amd as G
    from gptq_triton_amd import decoder_ops
    from gptq_triton_amd.llama import GreedyDecoder
    from test_loader import make_checkpoint
    cfg = make_checkpoint(tmp_path, 128, seed=21, act_order=act_order)
    model = G.load_quant(str(tmp_path), device="cuda", fuse_mlp=True)
    torch.manual_seed(5)
    ids = torch.randint(0, cfg.vocab_size, (bsz, 9)).cuda()
    monkeypatch.setattr(decoder_ops, "NORM_PAYS_ROWS", 4)   # by default only one-row steps take the 5-launch layer
    calls = []
    real = model.model.layers[0].mlp.forward_normed.__func__

    def spy(self, *a, **k):
        calls.append(1)
        return real(self, *a, **k)

    monkeypatch.setattr(type(model.model.layers[0].mlp), "forward_normed", spy)
    fused_eager = model.generate_greedy(ids, 10)
    assert len(calls) > 0, "the decode steps must have taken the fused-norm layer"
    fused_graph = model.generate_greedy(ids, 10, use_graph=True)
    monkeypatch.setattr(decoder_ops, "NORM_PAYS_ROWS", 0)
    n = len(calls)
    plain = model.generate_greedy(ids, 10)
    assert len(calls) == n, "with the fused norm switched off no call may reach it"
    assert torch.equal(fused_eager, plain) and torch.equal(fused_graph, plain)
