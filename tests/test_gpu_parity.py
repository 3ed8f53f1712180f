"""GPU parity: the HIP path (called through the C ABI via the ctypes binding) against
the CPU oracle on the same seeded inputs.

Bars: dequantised fp16 weights BIT-EXACT; matmul-type outputs within
|y - y_ref| <= 2e-3 + 1e-2 * |y_ref| of the oracle's wide-accumulation result
(the tolerance the task states), plus a much tighter sanity bound, since the kernels use
the same fp16 weights as the oracle and differ only in fp32 summation order and the
final fp16 rounding.
"""
import numpy as np
import pytest
import torch

from conftest import bits, to_dev
from oracle import gptq_oracle as O

pytestmark = pytest.mark.gpu

RTOL, ATOL = 1e-2, 2e-3


def assert_close(y, ref, what):
    y = np.asarray(y, dtype=np.float64)
    ok, max_abs, excess = O.within_tolerance(y, ref, RTOL, ATOL)
    assert ok, f"{what}: max_abs={max_abs:.3e} worst excess over tolerance={excess:.3e}"
    # tight bound: half an fp16 ulp of the result plus fp32 summation noise
    ref = np.asarray(ref, dtype=np.float64)
    ulp = np.spacing(np.abs(ref).astype(np.float16)).astype(np.float64)
    tight = 0.5 * ulp + 1e-4 * np.abs(ref) + 2e-4
    bad = np.abs(y - ref) > tight
    assert not bad.any(), f"{what}: {bad.sum()} elements beyond the tight bound, max_abs={max_abs:.3e}"


def gptq():
    import gptq_triton_amd
    return gptq_triton_amd


# ------------------------------------------------------------------ dequant (bit-exact)
@pytest.mark.parametrize("k,n,g,act", [(256, 256, 128, False), (4096, 4096, -1, False), (1024, 512, 128, True),
                                        (2048, 768, 256, True), (128, 8, -1, False)])
def test_dequant_bit_exact(k, n, g, act):
    L = O.make_layer(k, n, g, seed=11 + k + n, act_order=act)
    D = to_dev(L)
    w = gptq().dequantize(D["qweight"], D["qzeros"], D["scales"], k if g == -1 else g, D["g_idx"])
    ref = O.dequant_fp16(L["qweight"], L["qzeros"], L["scales"], g, L["g_idx"])
    assert (bits(w.cpu().numpy()) == bits(ref)).all()


def test_dequant_exhaustive_q_z_scale():
    """Every (q, z) pair against every fp16 scale in [0.002, 0.02], plus subnormal-range
    and large scales: column n has stored zero n % 16, row k has q = k % 16."""
    s_all = np.arange(np.float16(0.002).view(np.uint16), np.float16(0.02).view(np.uint16) + 1, dtype=np.uint16)
    extra = np.array([1e-7, 6e-8, 1e-5, 6.1e-5, 1.0, 3.0, 1000.0, 4000.0, 0.0], dtype=np.float16).view(np.uint16)
    s_vals = np.concatenate([s_all, extra]).view(np.float16)
    n = len(s_vals) * 16
    n = (n + 7) // 8 * 8
    scales = np.resize(np.repeat(s_vals, 16), n).astype(np.float16)[None, :]
    z = (np.arange(n) % 16).astype(np.uint8)[None, :]
    q = np.tile((np.arange(16) % 16).astype(np.uint8)[:, None], (1, n))
    L = dict(qweight=O.pack_qweight(q), qzeros=O.pack_qzeros(z), scales=scales)
    D = to_dev(L)
    w = gptq().dequantize(D["qweight"], D["qzeros"], D["scales"], 16)
    ref = O.dequant_fp16(L["qweight"], L["qzeros"], L["scales"], -1)
    assert (bits(w.cpu().numpy()) == bits(ref)).all()


def test_sort_rows_matches_gather():
    k, n, g = 1024, 256, 128
    L = O.make_layer(k, n, g, seed=5, act_order=True)
    D = to_dev(L)
    qs, perm = gptq().prepare_act_order(D["qweight"], D["g_idx"], g)
    perm_np = np.argsort(L["g_idx"], kind="stable")
    assert (perm.cpu().numpy() == perm_np).all()
    expect = O.pack_qweight(O.unpack_qweight(L["qweight"])[perm_np])
    assert (qs.cpu().numpy() == expect).all()


# ------------------------------------------------------------------------------ matmul
SHAPES = [(4096, 4096, -1), (4096, 4096, 128), (4096, 11008, 128), (11008, 4096, 128), (512, 256, 128),
          (128, 256, -1), (6656, 768, 512)]


@pytest.mark.parametrize("k,n,g", SHAPES)
@pytest.mark.parametrize("m", [1, 3, 16, 17, 100, 128, 300])
def test_matmul(k, n, g, m):
    L = O.make_layer(k, n, g, seed=k + n + m)
    x = O.make_x(m, k, seed=m)
    D = to_dev(L)
    y = gptq().matmul4(k if g == -1 else g, torch.from_numpy(x).cuda(), D["qweight"], D["scales"], D["qzeros"])
    ref = O.quant_matmul_ref(x, L["qweight"], L["qzeros"], L["scales"], g)
    assert y.shape == (m, n) and y.dtype == torch.float16
    assert_close(y.cpu().numpy(), ref, f"matmul K={k} N={n} g={g} M={m}")


@pytest.mark.parametrize("m", [1, 16, 64])
def test_matmul_bias_and_batch_dims(m):
    k, n, g = 1024, 512, 128
    L = O.make_layer(k, n, g, seed=3, bias=True)
    x = O.make_x(2 * m, k, seed=9).reshape(2, m, k)
    D = to_dev(L)
    y = gptq().matmul4(g, torch.from_numpy(x).cuda(), D["qweight"], D["scales"], D["qzeros"], D["bias"])
    assert y.shape == (2, m, n)
    ref16 = O.matmul_fp16(x, O.dequant_fp16(L["qweight"], L["qzeros"], L["scales"], g), L["bias"])
    ref = O.quant_matmul_ref(x, L["qweight"], L["qzeros"], L["scales"], g, bias=L["bias"])
    ok, max_abs, _ = O.within_tolerance(y.cpu().numpy(), ref)
    assert ok, max_abs
    # same rounding structure as the reference: fp16(acc) then an fp16 add of the bias
    # (the fp32 sums may differ in the last bit, so allow one ulp of the pre-bias value
    # plus one of the result)
    pre16 = O.matmul_fp16(x, O.dequant_fp16(L["qweight"], L["qzeros"], L["scales"], g))
    diff = np.abs(y.cpu().numpy().astype(np.float32) - ref16.astype(np.float32))
    lim = np.spacing(np.abs(ref16)).astype(np.float32) + np.spacing(np.abs(pre16)).astype(np.float32)
    assert (diff <= lim).all()


@pytest.mark.parametrize("m", [1, 16, 200])
def test_matmul_act_order(m):
    k, n, g = 2048, 512, 128
    L = O.make_layer(k, n, g, seed=21, act_order=True)
    x = O.make_x(m, k, seed=m + 1)
    G = gptq()
    layer = G.QuantLinear(4, g, k, n, bias=False, act_order=True)
    layer.qweight, layer.qzeros, layer.scales, layer.g_idx = (torch.from_numpy(L[t]) for t in
                                                               ("qweight", "qzeros", "scales", "g_idx"))
    layer = layer.cuda()
    y = layer(torch.from_numpy(x).cuda())
    ref = O.quant_matmul_ref(x, L["qweight"], L["qzeros"], L["scales"], g, g_idx=L["g_idx"])
    assert_close(y.cpu().numpy(), ref, f"act-order M={m}")
    # trivial g_idx reproduces the un-indexed result bit for bit
    layer2 = G.QuantLinear(4, g, k, n, bias=False, act_order=True)
    layer2.qweight, layer2.qzeros, layer2.scales = (torch.from_numpy(L[t]) for t in ("qweight", "qzeros", "scales"))
    layer2 = layer2.cuda()
    y2 = layer2(torch.from_numpy(x).cuda())
    y3 = G.matmul4(g, torch.from_numpy(x).cuda(), layer2.qweight, layer2.scales, layer2.qzeros)
    assert torch.equal(y2, y3)


def test_one_hot_rows_give_weight_rows_exactly():
    """x = e_k  =>  y = W[k, :] exactly (a single term, no summation error)."""
    k, n, g = 512, 256, 128
    L = O.make_layer(k, n, g, seed=8)
    W = O.dequant_fp16(L["qweight"], L["qzeros"], L["scales"], g)
    rows = [0, 7, 129, 511, 300, 64, 65, 8, 9, 255, 256, 383, 384, 100, 200, 501]
    x = np.zeros((len(rows), k), dtype=np.float16)
    for i, r in enumerate(rows):
        x[i, r] = 1.0
    D = to_dev(L)
    for m in (1, 5, 16):
        y = gptq().matmul4(g, torch.from_numpy(x[:m].copy()).cuda(), D["qweight"], D["scales"], D["qzeros"])
        assert (bits(y.cpu().numpy()) == bits(W[rows[:m]])).all()
    x32 = np.zeros((40, k), dtype=np.float16)
    for i in range(40):
        x32[i, (i * 13) % k] = 1.0
    y = gptq().matmul4(g, torch.from_numpy(x32).cuda(), D["qweight"], D["scales"], D["qzeros"])
    assert (bits(y.cpu().numpy()) == bits(W[[(i * 13) % k for i in range(40)]])).all()


@pytest.mark.parametrize("splitk", [1, 2, 3, 5, 8])
def test_splitk_variants_agree_and_counters_reset(splitk):
    from gptq_triton_amd import _lib
    k, n, g, m = 4096, 1024, 128, 4
    L = O.make_layer(k, n, g, seed=77)
    x = O.make_x(m, k, seed=78)
    D = to_dev(L)
    lib = _lib.load()
    ref = O.quant_matmul_ref(x, L["qweight"], L["qzeros"], L["scales"], g)
    try:
        lib.gptq4_set_tuning(0, 0, splitk)
        xd = torch.from_numpy(x).cuda()
        y1 = gptq().matmul4(g, xd, D["qweight"], D["scales"], D["qzeros"])
        y2 = gptq().matmul4(g, xd, D["qweight"], D["scales"], D["qzeros"])
    finally:
        lib.gptq4_set_tuning(0, 0, 0)
    assert torch.equal(y1, y2), "split-K result must be deterministic"
    assert_close(y1.cpu().numpy(), ref, f"splitk={splitk}")
    ws = _lib.workspace(xd.device, 0)
    torch.cuda.synchronize()
    assert int(ws[:_lib.WS_HEAD_BYTES].view(torch.int32).abs().sum()) == 0


# --------------------------------------------------------------------------- fused MLP
@pytest.mark.parametrize("g", [-1, 128])
@pytest.mark.parametrize("m", [1, 8, 16, 100, 256])
def test_mlp_gateup(g, m):
    k, n = 4096, 11008
    gate = O.make_layer(k, n, g, seed=100)
    up = O.make_layer(k, n, g, seed=101)
    x = O.make_x(m, k, seed=102 + m)
    Dg, Du = to_dev(gate), to_dev(up)
    gs = k if g == -1 else g
    h = gptq().llama_mlp_4(gs, torch.from_numpy(x).cuda(), Dg["qweight"], Dg["scales"], Dg["qzeros"],
                           Du["qweight"], Du["scales"], Du["qzeros"])
    ref = O.mlp_gateup_ref(x, (gate["qweight"], gate["qzeros"], gate["scales"]),
                           (up["qweight"], up["qzeros"], up["scales"]), g)
    assert_close(h.cpu().numpy(), ref, f"mlp gate/up g={g} M={m}")


@pytest.mark.parametrize("m", [1, 16, 40])
def test_mlp_module_end_to_end(m):
    k, n, g = 1024, 2816 - 2816 % 256, 128
    G = gptq()
    layers, raw = {}, {}
    for name, (ki, ni), seed in (("gate_proj", (k, n), 1), ("up_proj", (k, n), 2), ("down_proj", (n, k), 3)):
        L = O.make_layer(ki, ni, g, seed=seed)
        q = G.QuantLinear(4, g, ki, ni, bias=False)
        q.qweight, q.qzeros, q.scales = (torch.from_numpy(L[t]) for t in ("qweight", "qzeros", "scales"))
        layers[name], raw[name] = q, (L["qweight"], L["qzeros"], L["scales"])
    mlp = G.QuantLlamaMLP(layers["gate_proj"], layers["down_proj"], layers["up_proj"]).cuda()
    x = O.make_x(m, k, seed=50)
    xd = torch.from_numpy(x).cuda()
    y = mlp(xd).cpu().numpy()
    h = mlp.gate_up(xd).cpu().numpy()
    # (a) the fused gate/up stage against the oracle
    h_ref = O.mlp_gateup_ref(x, raw["gate_proj"], raw["up_proj"], g)
    assert_close(h, h_ref, f"mlp module gate/up M={m}")
    # (b) the down projection against the oracle fed with the SAME fp16 intermediate
    y_from_h = O.quant_matmul_ref(h, *raw["down_proj"], g)
    assert_close(y, y_from_h, f"mlp module down M={m}")
    # (c) the composed module against the composed oracle.  The fp16 intermediate can
    # round one ulp differently (fp32 vs float64 sums; |h| reaches ~90 with these
    # synthetic scales, so one ulp is up to 0.06); the oracle itself gives the exact
    # size of that effect, and nothing beyond it plus the stated tolerance is allowed.
    ref = O.mlp_ref(x, raw["gate_proj"], raw["up_proj"], raw["down_proj"], g)
    flips = (bits(h) != bits(h_ref.astype(np.float16))).mean()
    assert flips < 0.01
    err = np.abs(y.astype(np.float64) - ref)
    assert (err <= ATOL + RTOL * np.abs(ref) + np.abs(y_from_h - ref) + 1e-6).all()
    assert (np.abs(y_from_h - ref) <= 0.05).all()


# ------------------------------------------------------------------------ QKV + rotary
def test_rope_table_matches_closed_form():
    from gptq_triton_amd import RotaryTable
    cos, sin = RotaryTable(128, 2048, 10000.0).get(torch.device("cuda"), 2048)
    c_ref, s_ref = O.rotary_tables(2048, 128, 10000.0)
    assert np.abs(cos.cpu().numpy() - c_ref).max() <= 2e-7
    assert np.abs(sin.cpu().numpy() - s_ref).max() <= 2e-7


@pytest.mark.parametrize("b,s,pos0,g", [(1, 1, 2047, -1), (2, 5, 10, 128), (1, 300, 0, -1), (3, 1, 77, 128),
                                        (1, 16, 1000, -1), (1, 17, 0, 128),
                                        # tiled kernel: one token from each of 40 sequences; ragged S over several sequences
                                        (40, 1, 500, 128), (3, 43, 7, 128), (5, 130, 0, -1)])
def test_qkv_rotary(b, s, pos0, g):
    H, Dh, hidden = 8, 128, 1024
    L = O.make_layer(hidden, 3 * hidden, g, seed=200 + s)
    x = O.make_x(b * s, hidden, seed=201 + s).reshape(b, s, hidden)
    pos = (pos0 + np.arange(s))[None, :].repeat(b, 0)
    if b > 1:
        pos = pos + np.arange(b)[:, None] * 3
    D = to_dev(L)
    G = gptq()
    cos, sin = G.RotaryTable(Dh, 2048).get(torch.device("cuda"), 2048)
    q, k, v = G.qkv_rotary(hidden if g == -1 else g, torch.from_numpy(x).cuda(), D["qweight"], D["scales"],
                           D["qzeros"], torch.from_numpy(pos).cuda(), cos, sin, H, Dh)
    qr, kr, vr = O.qkv_rotary_ref(x, L["qweight"], L["qzeros"], L["scales"], g, pos, H, Dh, max_pos=2048)
    for got, ref, name in ((q, qr, "q"), (k, kr, "k"), (v, vr, "v")):
        assert got.shape == (b, H, s, Dh)
        assert_close(got.cpu().numpy(), ref, f"{name} b={b} s={s} g={g}")


def test_qkv_rotary_writes_into_kv_cache():
    H, Dh, hidden, g = 8, 128, 1024, 128
    L = O.make_layer(hidden, 3 * hidden, g, seed=300)
    D = to_dev(L)
    G = gptq()
    cos, sin = G.RotaryTable(Dh, 2048).get(torch.device("cuda"), 2048)
    cap = 40
    for s, off in ((20, 0), (1, 20), (18, 21)):
        x = O.make_x(2 * s, hidden, seed=301 + s).reshape(2, s, hidden)
        pos = (off + np.arange(s))[None, :].repeat(2, 0)
        kc = torch.full((2, H, cap, Dh), 7.0, dtype=torch.float16, device="cuda")
        vc = torch.full((2, H, cap, Dh), 7.0, dtype=torch.float16, device="cuda")
        xd, pd = torch.from_numpy(x).cuda(), torch.from_numpy(pos).cuda()
        q, k2, v2 = G.qkv_rotary(g, xd, D["qweight"], D["scales"], D["qzeros"], pd, cos, sin, H, Dh,
                                 kv_out=(kc, vc), kv_offset=off)
        q0, k0, v0 = G.qkv_rotary(g, xd, D["qweight"], D["scales"], D["qzeros"], pd, cos, sin, H, Dh)
        assert torch.equal(q, q0)
        assert torch.equal(kc[:, :, off:off + s], k0) and torch.equal(vc[:, :, off:off + s], v0)
        untouched = torch.ones(cap, dtype=torch.bool)
        untouched[off:off + s] = False
        assert bool((kc[:, :, untouched] == 7.0).all()) and bool((vc[:, :, untouched] == 7.0).all())


def test_qkv_rotary_places_rows_by_position_in_the_tiled_kernel():
    """kv_offset = KV_AT_POSITION with more than 16 rows: every token lands in the cache row of
    its own position id, whatever its place in the batch."""
    from gptq_triton_amd.fused_attention import KV_AT_POSITION
    H, Dh, hidden, g = 8, 128, 1024, 128
    L = O.make_layer(hidden, 3 * hidden, g, seed=320)
    D = to_dev(L)
    G = gptq()
    cos, sin = G.RotaryTable(Dh, 2048).get(torch.device("cuda"), 2048)
    b, s, cap = 3, 11, 64
    rng = np.random.default_rng(321)
    pos = np.stack([rng.permutation(cap)[:s] for _ in range(b)]).astype(np.int64)   # distinct rows per sequence
    x = O.make_x(b * s, hidden, seed=322).reshape(b, s, hidden)
    kc = torch.full((b, H, cap, Dh), 7.0, dtype=torch.float16, device="cuda")
    vc = torch.full((b, H, cap, Dh), 7.0, dtype=torch.float16, device="cuda")
    xd, pd = torch.from_numpy(x).cuda(), torch.from_numpy(pos).cuda()
    q, _, _ = G.qkv_rotary(g, xd, D["qweight"], D["scales"], D["qzeros"], pd, cos, sin, H, Dh,
                           kv_out=(kc, vc), kv_offset=KV_AT_POSITION)
    q0, k0, v0 = G.qkv_rotary(g, xd, D["qweight"], D["scales"], D["qzeros"], pd, cos, sin, H, Dh)
    assert torch.equal(q, q0)
    for bi in range(b):
        rows = torch.from_numpy(pos[bi]).cuda()
        assert torch.equal(kc[bi][:, rows], k0[bi]) and torch.equal(vc[bi][:, rows], v0[bi])
        untouched = torch.ones(cap, dtype=torch.bool)
        untouched[pos[bi]] = False
        assert bool((kc[bi][:, untouched] == 7.0).all()) and bool((vc[bi][:, untouched] == 7.0).all())


def test_fused_qkv_equals_three_projections():
    """Concatenation order q, k, v and column independence: the fused launch gives the
    same bits as three separate projections (cf. the reference's own fused-vs-unfused
    check, which asserts a zero difference)."""
    hidden, g = 1024, 128
    G = gptq()
    parts = [O.make_layer(hidden, hidden, g, seed=400 + i) for i in range(3)]
    fused = {t: np.concatenate([p[t] for p in parts], axis=1) for t in ("qweight", "qzeros", "scales")}
    for m in (1, 16, 64):
        x = torch.from_numpy(O.make_x(m, hidden, seed=410 + m)).cuda()
        Df = to_dev(fused)
        yf = G.matmul4(g, x, Df["qweight"], Df["scales"], Df["qzeros"])
        for i, p in enumerate(parts):
            Dp = to_dev(p)
            yp = G.matmul4(g, x, Dp["qweight"], Dp["scales"], Dp["qzeros"])
            if m > 16:
                assert torch.equal(yf[:, i * hidden:(i + 1) * hidden], yp)
            else:
                # the split-K factor depends on N, so the fp32 summation order may differ
                d = (yf[:, i * hidden:(i + 1) * hidden].float() - yp.float()).abs().max().item()
                assert d <= 2 ** -7


@pytest.mark.parametrize("own_gather", [False, True])
def test_act_order_above_16_rows_staged_or_gathered_by_the_tiled_kernel(own_gather):
    """With `perm` the call gathers the rows of x into its workspace and runs the plain kernels; asked to
    (tile selector + 10), the tiled kernel gathers in its own A staging instead.  Same result either way."""
    from gptq_triton_amd import _lib
    k, n, g, m = 1024, 512, 128, 40
    L = O.make_layer(k, n, g, seed=31, act_order=True)
    x = O.make_x(m, k, seed=32)
    G = gptq()
    qs, perm = G.prepare_act_order(torch.from_numpy(L["qweight"]).cuda(), torch.from_numpy(L["g_idx"]).cuda(), g)
    D = to_dev(L)
    xd = torch.from_numpy(x).cuda()
    y = torch.empty((m, n), dtype=torch.float16, device="cuda")
    lib = _lib.load()
    ws = _lib.workspace(xd.device, lib.gptq4_workspace_bytes(_lib.OP_MATMUL | _lib.OP_WITH_PERM, m, k, n))
    if own_gather:
        lib.gptq4_set_midm_tuning(0, 0, 0)
        lib.gptq4_set_gemm_tuning(10, 0)
    try:
        rc = lib.gptq4_matmul(xd.data_ptr(), qs.data_ptr(), D["qzeros"].data_ptr(), D["scales"].data_ptr(), perm.data_ptr(),
                              None, y.data_ptr(), m, k, n, g, ws.data_ptr(), ws.numel(), _lib.current_stream(xd.device))
    finally:
        lib.gptq4_set_gemm_tuning(0, 0)
        lib.gptq4_set_midm_tuning(1, 0, 0)
    assert rc == 0
    ref = O.quant_matmul_ref(x, L["qweight"], L["qzeros"], L["scales"], g, g_idx=L["g_idx"])
    assert_close(y.cpu().numpy(), ref, f"act-order, M={m}, own gather {own_gather}")


@pytest.mark.parametrize("k,n", [(128, 256), (640, 768), (1408, 512), (3072, 1024)])
@pytest.mark.parametrize("m", [1, 3, 16, 17, 77, 300, 600])
def test_a_call_with_perm_equals_the_call_on_gathered_rows(k, n, m):
    """Whatever kernel the row count selects, passing `perm` must give the very bits of the same call on
    x[:, perm]: the call only gathers the rows (for the decode GEMV: inside its LDS copy) and then does what it
    does without a permutation.  Odd K included (K/128 = 1, 5, 11, 24)."""
    G = gptq()
    gen = torch.Generator(device="cuda"); gen.manual_seed(k + n + m)
    g = 128
    W = [(torch.randint(-2**31, 2**31 - 1, (k // 8, n), dtype=torch.int32, device="cuda", generator=gen),
          torch.randint(-2**31, 2**31 - 1, (k // g, n // 8), dtype=torch.int32, device="cuda", generator=gen),
          (0.002 + 0.02 * torch.rand((k // g, n), device="cuda", generator=gen)).half()) for _ in range(2)]
    perm = torch.randperm(k, device="cuda", generator=gen).int()
    x = torch.randn((m, k), device="cuda", generator=gen).half()
    xg = x[:, perm.long()].contiguous()
    (q0, z0, s0), (q1, z1, s1) = W
    assert torch.equal(G.matmul4(g, x, q0, s0, z0, perm=perm), G.matmul4(g, xg, q0, s0, z0))
    assert torch.equal(G.llama_mlp_4(g, x, q0, s0, z0, q1, s1, z1, perm=perm), G.llama_mlp_4(g, xg, q0, s0, z0, q1, s1, z1))


@pytest.mark.parametrize("heads", [2, 6, 10])
@pytest.mark.parametrize("m", [1, 3, 16, 17, 77, 300, 600])
def test_qkv_rotary_with_perm_equals_the_call_on_gathered_rows(heads, m):
    G = gptq()
    gen = torch.Generator(device="cuda"); gen.manual_seed(heads + m)
    k, g = heads * 128, 128
    qw = torch.randint(-2**31, 2**31 - 1, (k // 8, 3 * k), dtype=torch.int32, device="cuda", generator=gen)
    qz = torch.randint(-2**31, 2**31 - 1, (k // g, 3 * k // 8), dtype=torch.int32, device="cuda", generator=gen)
    sc = (0.002 + 0.02 * torch.rand((k // g, 3 * k), device="cuda", generator=gen)).half()
    perm = torch.randperm(k, device="cuda", generator=gen).int()
    x = torch.randn((1, m, k), device="cuda", generator=gen).half()
    xg = x[..., perm.long()].contiguous()
    cos, sin = G.RotaryTable(128, 1024).get(torch.device("cuda"), 1024)
    pos = torch.arange(m, device="cuda", dtype=torch.int32)[None]
    a = G.qkv_rotary(g, x, qw, sc, qz, pos, cos, sin, heads, perm=perm)
    b = G.qkv_rotary(g, xg, qw, sc, qz, pos, cos, sin, heads)
    assert all(torch.equal(u, v) for u, v in zip(a, b))


def test_empty_inputs_give_empty_outputs():
    """Zero rows: every functional returns a tensor of the right shape and launches nothing;
    the C entry points themselves reject M < 1."""
    from gptq_triton_amd import _lib
    k, n, g = 256, 512, 128
    L = O.make_layer(k, n, g, seed=900)
    D = to_dev(L)
    G = gptq()
    x0 = torch.empty((0, k), dtype=torch.float16, device="cuda")
    assert G.matmul4(g, x0, D["qweight"], D["scales"], D["qzeros"]).shape == (0, n)
    assert G.matmul4(g, x0.view(2, 0, k), D["qweight"], D["scales"], D["qzeros"]).shape == (2, 0, n)
    assert G.llama_mlp_4(g, x0, D["qweight"], D["scales"], D["qzeros"], D["qweight"], D["scales"], D["qzeros"]).shape == (0, n)
    Lq = O.make_layer(256, 768, g, seed=901)
    Dq = to_dev(Lq)
    cos, sin = G.RotaryTable(128, 64).get(torch.device("cuda"), 64)
    pos0 = torch.empty((1, 0), dtype=torch.int64, device="cuda")
    q, kk, vv = G.qkv_rotary(g, x0.view(1, 0, k), Dq["qweight"], Dq["scales"], Dq["qzeros"], pos0, cos, sin, 2, 128)
    assert q.shape == kk.shape == vv.shape == (1, 2, 0, 128)
    lib = _lib.load()
    ws = _lib.workspace(x0.device, lib.gptq4_workspace_bytes(_lib.OP_MATMUL, 1, k, n))
    y = torch.empty((1, n), dtype=torch.float16, device="cuda")
    x1 = torch.zeros((1, k), dtype=torch.float16, device="cuda")
    rc = lib.gptq4_matmul(x1.data_ptr(), D["qweight"].data_ptr(), D["qzeros"].data_ptr(), D["scales"].data_ptr(), None, None,
                          y.data_ptr(), 0, k, n, g, ws.data_ptr(), ws.numel(), _lib.current_stream(x0.device))
    assert rc < 0 and b"shape" in lib.gptq4_strerror(rc).lower()


@pytest.mark.parametrize("words,depth", [(1, 2), (1, 4), (2, 1), (2, 2), (2, 4), (4, 1), (4, 2)])
@pytest.mark.parametrize("act_order", [False, True])
@pytest.mark.parametrize("m", [1, 7, 16])
def test_split_k_kernel_launch_shapes(words, depth, act_order, m):
    """Every load width (4, 8, 16 bytes per lane) and ring depth of the split-K decode kernel, all three
    epilogues, with and without act-order, with the balanced GEMV switched off so that the calls reach it."""
    from gptq_triton_amd import _lib
    G = gptq()
    lib = _lib.load()
    k, n, g, heads = 1024, 768, 128, 8   # the oracle's rotary path wants hidden = heads * 128
    gate = O.make_layer(k, n, g, seed=40 + words, act_order=act_order, bias=True)
    up = O.make_layer(k, n, g, seed=41 + words)
    up["g_idx"] = gate["g_idx"]
    qkv = O.make_layer(k, 3 * k, g, seed=42 + words)
    qkv["g_idx"] = gate["g_idx"]
    x = O.make_x(m, k, seed=43 + m)
    xd = torch.from_numpy(x).cuda()
    Dg, Du, Dq = to_dev(gate), to_dev(up), to_dev(qkv)
    gq, uq, qq, perm = Dg["qweight"], Du["qweight"], Dq["qweight"], None
    if act_order:
        gq, perm = G.prepare_act_order(Dg["qweight"], Dg["g_idx"], g)
        uq, _ = G.prepare_act_order(Du["qweight"], Dg["g_idx"], g)
        qq, _ = G.prepare_act_order(Dq["qweight"], Dg["g_idx"], g)
    cos, sin = G.RotaryTable(128, 64).get(torch.device("cuda"), 64)
    pos = (np.arange(m) % 50)[:, None].astype(np.int32)
    lib.gptq4_set_gemv_tuning(0, 0, 0, 0)
    lib.gptq4_set_tuning(words, depth, 0)
    try:
        y = G.matmul4(g, xd, gq, Dg["scales"], Dg["qzeros"], Dg["bias"], perm=perm)
        h = G.llama_mlp_4(g, xd, gq, Dg["scales"], Dg["qzeros"], uq, Du["scales"], Du["qzeros"], perm=perm)
        q, kk, vv = G.qkv_rotary(g, xd.view(m, 1, k), qq, Dq["scales"], Dq["qzeros"], torch.from_numpy(pos).cuda(),
                                 cos, sin, heads, perm=perm)
    finally:
        lib.gptq4_set_tuning(0, 0, 0)
        lib.gptq4_set_gemv_tuning(1, 0, 0, 0)
    gi = gate["g_idx"]
    ref = O.quant_matmul_ref(x, gate["qweight"], gate["qzeros"], gate["scales"], g, bias=gate["bias"], g_idx=gi)
    ok, max_abs, _ = O.within_tolerance(y.cpu().numpy(), ref)
    assert ok, max_abs
    href = O.mlp_gateup_ref(x, (gate["qweight"], gate["qzeros"], gate["scales"], gi), (up["qweight"], up["qzeros"], up["scales"], gi), g)
    assert_close(h.cpu().numpy(), href, f"gate/up words={words} depth={depth} M={m}")
    qr, kr, vr = O.qkv_rotary_ref(x.reshape(m, 1, k), qkv["qweight"], qkv["qzeros"], qkv["scales"], g, pos, heads, 128,
                                  g_idx=gi, max_pos=64)
    for got, want, name in ((q, qr, "q"), (kk, kr, "k"), (vv, vr, "v")):
        assert_close(got.cpu().numpy(), want, f"{name} words={words} depth={depth} M={m}")
