"""GPU parity of the balanced decode GEMV, forced on for every shape it accepts (by default
it only serves the one-row gate/up pair): rows 1..4, all
three epilogues, act-order, bias, tiny and ragged unit counts, several launch shapes.
Same bars as test_gpu_parity.py."""
import numpy as np
import pytest
import torch

from conftest import to_dev
from oracle import gptq_oracle as O
from test_gpu_parity import assert_close, gptq

pytestmark = pytest.mark.gpu

# (units in flight, waves per workgroup, waves per CU); 0 = automatic
CONFIGS = [(0, 0, 0), (3, 8, 16), (2, 16, 16), (2, 8, 4), (1, 8, 8), (2, 4, 8), (3, 4, 8)]


@pytest.fixture(params=CONFIGS, ids=lambda c: "d%d_w%d_cu%d" % c)
def forced_gemv(request):
    from gptq_triton_amd import _lib
    lib = _lib.load()
    lib.gptq4_set_gemv_tuning(2, *request.param)
    yield lib
    lib.gptq4_set_gemv_tuning(1, 0, 0, 0)


@pytest.mark.parametrize("k,n,g", [(4096, 1024, 128), (1408, 512, -1), (128, 256, 128), (2048, 256, 512)])
@pytest.mark.parametrize("m", [1, 2, 3, 4])
def test_gemv_matmul(forced_gemv, k, n, g, m):
    L = O.make_layer(k, n, g, seed=k + n + m, bias=(m % 2 == 0))
    x = O.make_x(m, k, seed=m + 5)
    D = to_dev(L)
    xd = torch.from_numpy(x).cuda()
    y = gptq().matmul4(k if g == -1 else g, xd, D["qweight"], D["scales"], D["qzeros"], D.get("bias"))
    y2 = gptq().matmul4(k if g == -1 else g, xd, D["qweight"], D["scales"], D["qzeros"], D.get("bias"))
    assert torch.equal(y, y2), "the slot-ordered reduction must be deterministic"
    ref = O.quant_matmul_ref(x, L["qweight"], L["qzeros"], L["scales"], g, bias=L["bias"])
    if L["bias"] is None:
        assert_close(y.cpu().numpy(), ref, f"gemv matmul K={k} N={n} g={g} M={m}")
    else:
        ok, max_abs, _ = O.within_tolerance(y.cpu().numpy(), ref)
        assert ok, max_abs


def test_gemv_leaves_the_workspace_head_zero(forced_gemv):
    from gptq_triton_amd import _lib
    k, n, g = 4096, 1024, 128
    L = O.make_layer(k, n, g, seed=1)
    D = to_dev(L)
    xd = torch.from_numpy(O.make_x(3, k, seed=2)).cuda()
    gptq().matmul4(g, xd, D["qweight"], D["scales"], D["qzeros"])
    ws = _lib.workspace(xd.device, 0)
    torch.cuda.synchronize()
    assert int(ws[:_lib.WS_HEAD_BYTES].view(torch.int32).abs().sum()) == 0


@pytest.mark.parametrize("m", [1, 4])
def test_gemv_act_order(forced_gemv, m):
    k, n, g = 2048, 512, 128
    L = O.make_layer(k, n, g, seed=21, act_order=True)
    x = O.make_x(m, k, seed=m + 1)
    G = gptq()
    layer = G.QuantLinear(4, g, k, n, bias=False, act_order=True)
    layer.qweight, layer.qzeros, layer.scales, layer.g_idx = (torch.from_numpy(L[t]) for t in
                                                               ("qweight", "qzeros", "scales", "g_idx"))
    y = layer.cuda()(torch.from_numpy(x).cuda())
    ref = O.quant_matmul_ref(x, L["qweight"], L["qzeros"], L["scales"], g, g_idx=L["g_idx"])
    assert_close(y.cpu().numpy(), ref, f"gemv act-order M={m}")


@pytest.mark.parametrize("m", [1, 4])
def test_gemv_act_order_fused_epilogues(forced_gemv, m):
    """Act-order under the SiLU*mul and the rotary epilogue: the waves gather their x slices through perm."""
    G = gptq()
    k, n, g, heads = 1024, 768, 128, 8
    gate = O.make_layer(k, n, g, seed=60, act_order=True)
    up = O.make_layer(k, n, g, seed=61)
    qkv = O.make_layer(k, 3 * k, g, seed=62)
    up["g_idx"] = qkv["g_idx"] = gate["g_idx"]
    Dg, Du, Dq = to_dev(gate), to_dev(up), to_dev(qkv)
    gq, perm = G.prepare_act_order(Dg["qweight"], Dg["g_idx"], g)
    uq, _ = G.prepare_act_order(Du["qweight"], Dg["g_idx"], g)
    qq, _ = G.prepare_act_order(Dq["qweight"], Dg["g_idx"], g)
    x = O.make_x(m, k, seed=63 + m)
    xd = torch.from_numpy(x).cuda()
    h = G.llama_mlp_4(g, xd, gq, Dg["scales"], Dg["qzeros"], uq, Du["scales"], Du["qzeros"], perm=perm)
    gi = gate["g_idx"]
    href = O.mlp_gateup_ref(x, (gate["qweight"], gate["qzeros"], gate["scales"], gi), (up["qweight"], up["qzeros"], up["scales"], gi), g)
    assert_close(h.cpu().numpy(), href, f"gemv act-order gate/up M={m}")
    cos, sin = G.RotaryTable(128, 2048).get(torch.device("cuda"), 2048)
    pos = (np.arange(m) * 7 + 3)[:, None].astype(np.int32)
    q, kk, vv = G.qkv_rotary(g, xd.view(m, 1, k), qq, Dq["scales"], Dq["qzeros"], torch.from_numpy(pos).cuda(), cos, sin, heads, perm=perm)
    qr, kr, vr = O.qkv_rotary_ref(x.reshape(m, 1, k), qkv["qweight"], qkv["qzeros"], qkv["scales"], g, pos, heads, 128, g_idx=gi, max_pos=2048)
    for got, want, name in ((q, qr, "q"), (kk, kr, "k"), (vv, vr, "v")):
        assert_close(got.cpu().numpy(), want, f"gemv act-order {name} M={m}")


@pytest.mark.parametrize("g", [-1, 128])
@pytest.mark.parametrize("m", [1, 3])
def test_gemv_gateup(forced_gemv, g, m):
    k, n = 1024, 2816
    gate = O.make_layer(k, n, g, seed=100)
    up = O.make_layer(k, n, g, seed=101)
    x = O.make_x(m, k, seed=102 + m)
    Dg, Du = to_dev(gate), to_dev(up)
    h = gptq().llama_mlp_4(k if g == -1 else g, torch.from_numpy(x).cuda(), Dg["qweight"], Dg["scales"], Dg["qzeros"],
                           Du["qweight"], Du["scales"], Du["qzeros"])
    ref = O.mlp_gateup_ref(x, (gate["qweight"], gate["qzeros"], gate["scales"]),
                           (up["qweight"], up["qzeros"], up["scales"]), g)
    assert_close(h.cpu().numpy(), ref, f"gemv gate/up g={g} M={m}")


@pytest.mark.parametrize("b,s,pos0,g", [(1, 1, 2047, -1), (2, 2, 10, 128), (1, 4, 1000, 128), (3, 1, 77, -1)])
def test_gemv_qkv_rotary(forced_gemv, b, s, pos0, g):
    H, Dh, hidden = 8, 128, 1024
    L = O.make_layer(hidden, 3 * hidden, g, seed=200 + s)
    x = O.make_x(b * s, hidden, seed=201 + s).reshape(b, s, hidden)
    pos = (pos0 + np.arange(s))[None, :].repeat(b, 0) + np.arange(b)[:, None] * 3
    D = to_dev(L)
    G = gptq()
    cos, sin = G.RotaryTable(Dh, 2048).get(torch.device("cuda"), 2048)
    q, k, v = G.qkv_rotary(hidden if g == -1 else g, torch.from_numpy(x).cuda(), D["qweight"], D["scales"],
                           D["qzeros"], torch.from_numpy(pos).cuda(), cos, sin, H, Dh)
    qr, kr, vr = O.qkv_rotary_ref(x, L["qweight"], L["qzeros"], L["scales"], g, pos, H, Dh, max_pos=2048)
    for got, ref, name in ((q, qr, "q"), (k, kr, "k"), (v, vr, "v")):
        assert_close(got.cpu().numpy(), ref, f"gemv {name} b={b} s={s} g={g}")


def test_gemv_and_splitk_kernels_agree_within_rounding():
    """The two small-M kernels sum the same fp16 products in different fp32 orders."""
    from gptq_triton_amd import _lib
    lib = _lib.load()
    k, n, g = 4096, 4096, 128
    L = O.make_layer(k, n, g, seed=5)
    D = to_dev(L)
    xd = torch.from_numpy(O.make_x(1, k, seed=6)).cuda()
    try:
        lib.gptq4_set_gemv_tuning(0, 0, 0, 0)
        y0 = gptq().matmul4(g, xd, D["qweight"], D["scales"], D["qzeros"]).float()
        lib.gptq4_set_gemv_tuning(2, 0, 0, 0)
        y1 = gptq().matmul4(g, xd, D["qweight"], D["scales"], D["qzeros"]).float()
    finally:
        lib.gptq4_set_gemv_tuning(1, 0, 0, 0)
    big = torch.maximum(y0.abs(), y1.abs()).cpu().numpy().astype(np.float16)
    ulp = torch.from_numpy(np.spacing(big).astype(np.float32)).cuda()
    # one fp16 step of the result, plus fp32 summation noise where the sum nearly cancels
    assert bool(((y0 - y1).abs() <= ulp + 1e-4).all())
