"""GPU parity of the streaming-order layout and its decode kernel (gptq4_stream_*), through the C ABI.

Bars as elsewhere: layout conversions and dequantised weights BIT-EXACT (the conversions against the oracle's
word-by-word definition, the dequantisation against the oracle's formula); matmul-type outputs within
|y - y_ref| <= 2e-3 + 1e-2 * |y_ref| of the float64 oracle and within the tight bound of test_gpu_parity; the variants
that normalise their own input bit-identical to the norm launch followed by the plain call; results equal from run to
run and the head of the workspace zero after every call.
"""
import numpy as np
import pytest
import torch

from conftest import bits, to_dev
from oracle import gptq_oracle as O
from test_gpu_parity import assert_close

pytestmark = pytest.mark.gpu


def gptq():
    import gptq_triton_amd
    return gptq_triton_amd


def lib_():
    from gptq_triton_amd import _lib
    return _lib


def head_is_zero():
    _lib = lib_()
    torch.cuda.synchronize()
    return all(int(ws[:_lib.WS_HEAD_BYTES].view(torch.int64).abs().sum()) == 0 for ws in _lib._workspaces.values())


SHAPES = [(1024, 256, 128), (1024, 512, -1), (4096, 4096, 128), (4096, 4096, -1), (11008, 4096, 128), (2048, 768, 512),
          (5120, 5120, 128), (6656, 6656, 512), (4096, 12288, 128)]


# ------------------------------------------------------------------ the layout itself
@pytest.mark.parametrize("k,n,g", [(1024, 256, 128), (2048, 768, 512), (4096, 4096, -1), (128, 256, -1)])
def test_pack_matches_the_definition_and_round_trips(k, n, g):
    G = gptq()
    L = O.make_layer(k, n, g, seed=900 + k)
    D = to_dev(L)
    sw, meta = G.stream_pack(D["qweight"], D["qzeros"], D["scales"], g)
    ref_sw, ref_meta = O.stream_order(L["qweight"], L["qzeros"], L["scales"])
    if k * n <= 1024 * 256:
        assert (O.stream_order_loops(L["qweight"]) == ref_sw).all()
    assert (sw.cpu().numpy() == ref_sw).all() and (meta.cpu().numpy() == ref_meta).all()
    assert torch.equal(G.stream_unpack(sw), D["qweight"])
    # the torch implementation used off the GPU (a model moved to the CPU to be saved) gives the same words
    sw_cpu, meta_cpu = G.stream_pack(D["qweight"].cpu(), D["qzeros"].cpu(), D["scales"].cpu(), g)
    assert torch.equal(sw_cpu, sw.cpu()) and torch.equal(meta_cpu, meta.cpu())
    assert torch.equal(G.stream_unpack(sw_cpu), D["qweight"].cpu())
    # the full inverse through the C ABI: qzeros and scales back as well
    _lib = lib_()
    lib = _lib.load()
    qw2, qz2, sc2 = torch.empty_like(D["qweight"]), torch.empty_like(D["qzeros"]), torch.empty_like(D["scales"])
    rc = lib.gptq4_stream_unpack(sw.data_ptr(), meta.data_ptr(), qw2.data_ptr(), qz2.data_ptr(), sc2.data_ptr(), k, n, g,
                                 _lib.current_stream(sw.device))
    assert rc == 0
    assert torch.equal(qw2, D["qweight"]) and torch.equal(qz2, D["qzeros"]) and torch.equal(sc2.view(torch.int16), D["scales"].view(torch.int16))


@pytest.mark.parametrize("k,n,g", [(256, 256, 128), (4096, 4096, -1), (2048, 768, 256), (1024, 512, 128)])
def test_dequant_from_the_streaming_order_is_bit_exact(k, n, g):
    G = gptq()
    _lib = lib_()
    L = O.make_layer(k, n, g, seed=910 + n)
    D = to_dev(L)
    sw, meta = G.stream_pack(D["qweight"], D["qzeros"], D["scales"], g)
    w = torch.empty((k, n), dtype=torch.float16, device="cuda")
    assert _lib.load().gptq4_stream_dequant(sw.data_ptr(), meta.data_ptr(), w.data_ptr(), k, n, g, _lib.current_stream(w.device)) == 0
    ref = O.dequant_fp16(L["qweight"], L["qzeros"], L["scales"], g)
    assert (bits(w.cpu().numpy()) == bits(ref)).all()


def test_dequant_from_the_streaming_order_exhaustive_q_z_scale():
    """Every (q, z) pair against every fp16 scale in [0.002, 0.02] plus subnormal-range and large scales, through
    the {scale, zero} words of the streaming order."""
    G = gptq()
    _lib = lib_()
    s_all = np.arange(np.float16(0.002).view(np.uint16), np.float16(0.02).view(np.uint16) + 1, dtype=np.uint16)
    extra = np.array([1e-7, 6e-8, 1e-5, 6.1e-5, 1.0, 3.0, 1000.0, 4000.0, 0.0], dtype=np.float16).view(np.uint16)
    s_vals = np.concatenate([s_all, extra]).view(np.float16)
    n = (len(s_vals) * 16 + 255) // 256 * 256
    k = 128
    scales = np.resize(np.repeat(s_vals, 16), n).astype(np.float16)[None, :]
    z = (np.arange(n) % 16).astype(np.uint8)[None, :]
    q = np.tile((np.arange(k) % 16).astype(np.uint8)[:, None], (1, n))
    L = dict(qweight=O.pack_qweight(q), qzeros=O.pack_qzeros(z), scales=scales)
    D = to_dev(L)
    sw, meta = G.stream_pack(D["qweight"], D["qzeros"], D["scales"], -1)
    w = torch.empty((k, n), dtype=torch.float16, device="cuda")
    assert _lib.load().gptq4_stream_dequant(sw.data_ptr(), meta.data_ptr(), w.data_ptr(), k, n, -1, _lib.current_stream(w.device)) == 0
    assert (bits(w.cpu().numpy()) == bits(O.dequant_fp16(L["qweight"], L["qzeros"], L["scales"], -1))).all()


# ------------------------------------------------------------------ the three operators
@pytest.mark.parametrize("k,n,g", SHAPES)
@pytest.mark.parametrize("m", [1, 2, 3, 4, 5, 8, 13, 16])
def test_matmul(k, n, g, m):
    G = gptq()
    L = O.make_layer(k, n, g, seed=1000 + k + n, bias=(m == 2))
    D = to_dev(L)
    gs = k if g == -1 else g
    if G.quant_linear.stream_rows(0, k, n, gs) < m:
        pytest.skip("shape outside what the streaming-order kernel takes")
    sw, meta = G.stream_pack(D["qweight"], D["qzeros"], D["scales"], gs)
    x = O.make_x(m, k, seed=m + 3)
    xd = torch.from_numpy(x).cuda()
    y = G.matmul4_stream(gs, xd, sw, meta, D.get("bias"))
    ref = O.quant_matmul_ref(x, L["qweight"], L["qzeros"], L["scales"], g, bias=L.get("bias"))
    if L.get("bias") is None:
        assert_close(y.cpu().numpy(), ref, f"stream matmul {k}x{n} g={g} M={m}")
    else:
        ok, max_abs, _ = O.within_tolerance(y.cpu().numpy(), ref)
        assert ok, max_abs
        # the reference's rounding structure (quant_linear.py:225,280-281): fp16(acc), then an fp16 add of the bias - two
        # roundings, so one ulp of the value before the bias plus one of the result
        w = O.dequant_fp16(L["qweight"], L["qzeros"], L["scales"], g)
        ref16, pre16 = O.matmul_fp16(x, w, L["bias"]), O.matmul_fp16(x, w)
        diff = np.abs(y.cpu().numpy().astype(np.float32) - ref16.astype(np.float32))
        assert (diff <= np.spacing(np.abs(ref16)).astype(np.float32) + np.spacing(np.abs(pre16)).astype(np.float32)).all()
    assert torch.equal(G.matmul4_stream(gs, xd, sw, meta, D.get("bias")), y), "results must not change from run to run"
    assert head_is_zero()


@pytest.mark.parametrize("k,n,g", [(1024, 512, 128), (4096, 4096, -1), (11008, 4096, 128), (4096, 12288, 128)])
@pytest.mark.parametrize("m", [17, 100, 640, 2048])
def test_matmul_with_more_rows_reads_the_same_words(k, n, g, m):
    """Above 16 rows the tiled kernel reads the streaming order itself (no copy in the checkpoint order is made)."""
    G = gptq()
    L = O.make_layer(k, n, g, seed=1600 + k + m, bias=(m == 100))
    D = to_dev(L)
    gs = k if g == -1 else g
    sw, meta = G.stream_pack(D["qweight"], D["qzeros"], D["scales"], gs)
    x = O.make_x(m, k, seed=m)
    y = G.matmul4_stream(gs, torch.from_numpy(x).cuda(), sw, meta, D.get("bias"))
    rows = np.unique(np.concatenate([[r for r in (0, 1, 16, 31, 32, m - 1) if r < m], np.random.default_rng(m).choice(m, size=min(m, 12), replace=False)]))
    ref = O.quant_matmul_ref(x[rows], L["qweight"], L["qzeros"], L["scales"], g, bias=L.get("bias"))
    ok, max_abs, _ = O.within_tolerance(y[rows].cpu().numpy(), ref)
    assert ok, max_abs
    if L.get("bias") is None:
        assert_close(y[rows].cpu().numpy(), ref, f"tiled kernel on streaming order {k}x{n} M={m}")
    assert head_is_zero()


@pytest.mark.parametrize("m", [48, 2048])
def test_fused_operators_with_more_rows_read_the_same_words(m):
    G = gptq()
    k, inter, heads, g = 1024, 2816, 8, 128
    gate, up = O.make_layer(k, inter, g, seed=1700), O.make_layer(k, inter, g, seed=1701)
    Dg, Du = to_dev(gate), to_dev(up)
    gsw, gm = G.stream_pack(Dg["qweight"], Dg["qzeros"], Dg["scales"], g)
    usw, um = G.stream_pack(Du["qweight"], Du["qzeros"], Du["scales"], g)
    x = O.make_x(m, k, seed=m + 1)
    xd = torch.from_numpy(x).cuda()
    rows = np.unique(np.concatenate([[0, 31, 32, m - 1], np.random.default_rng(m).choice(m, size=10, replace=False)]))
    y = G.llama_mlp_4_stream(g, xd, gsw, gm, usw, um)
    trip = lambda d: (d["qweight"], d["qzeros"], d["scales"])
    assert_close(y[rows].cpu().numpy(), O.mlp_gateup_ref(x[rows], trip(gate), trip(up), g), f"tiled gate/up on streaming order M={m}")
    # fused QKV + rotary, two sequences
    L = O.make_layer(k, 3 * heads * 128, g, seed=1702)
    D = to_dev(L)
    sw, meta = G.stream_pack(D["qweight"], D["qzeros"], D["scales"], g)
    b, s = 2, m // 2
    x3 = x.reshape(b, s, k)
    pos = (np.arange(s, dtype=np.int64)[None, :] + np.array([[3], [40]]))
    cos, sin = G.RotaryTable(128, 4096).get(torch.device("cuda"), 4096)
    q, kk, vv = G.qkv_rotary_stream(g, torch.from_numpy(x3).cuda(), sw, meta, torch.from_numpy(pos).cuda(), cos, sin, heads)
    q2, k2, v2 = G.qkv_rotary(g, torch.from_numpy(x3).cuda(), D["qweight"], D["scales"], D["qzeros"], torch.from_numpy(pos).cuda(), cos, sin, heads)
    toks = np.unique(np.concatenate([[0, s - 1], np.random.default_rng(s).choice(s, size=6, replace=False)]))
    qr, kr, vr = O.qkv_rotary_ref(x3[:, toks], L["qweight"], L["qzeros"], L["scales"], g, pos[:, toks], heads, max_pos=4096)
    for got, ref, name in ((q, qr, "q"), (kk, kr, "k"), (vv, vr, "v")):
        assert_close(got[:, :, toks].cpu().numpy(), ref, f"tiled qkv {name} on streaming order M={m}")
    assert head_is_zero()


@pytest.mark.parametrize("m", [17, 32, 33, 64, 128, 256, 300, 512])
def test_mid_sized_calls_at_llama7b_shapes_agree_with_the_checkpoint_order_kernels(m):
    """17 .. a few hundred rows: the K-sliced kernel (whole and paired rotary heads, 64- and 128-column strips, four and
    eight waves, K split across workgroups) reads the streaming order too; same values as from the checkpoint order up
    to the order of the fp32 sums, and the oracle's on sampled rows."""
    G = gptq()
    H, I, heads, g = 4096, 11008, 32, 128
    rows = np.unique(np.concatenate([[0, m - 1], np.random.default_rng(m).choice(m, size=min(m, 6), replace=False)]))
    x = O.make_x(m, H, seed=m + 7)
    xd = torch.from_numpy(x).cuda()
    trip = lambda d: (d["qweight"], d["qzeros"], d["scales"])
    # gate/up
    gate, up = O.make_layer(H, I, g, seed=1800), O.make_layer(H, I, g, seed=1801)
    Dg, Du = to_dev(gate), to_dev(up)
    gsw, gm = G.stream_pack(Dg["qweight"], Dg["qzeros"], Dg["scales"], g)
    usw, um = G.stream_pack(Du["qweight"], Du["qzeros"], Du["scales"], g)
    ys = G.llama_mlp_4_stream(g, xd, gsw, gm, usw, um)
    yc = G.llama_mlp_4(g, xd, Dg["qweight"], Dg["scales"], Dg["qzeros"], Du["qweight"], Du["scales"], Du["qzeros"])
    ok, max_abs, _ = O.within_tolerance(ys.cpu().numpy(), yc.float().cpu().numpy())
    assert ok, max_abs
    assert_close(ys[rows].cpu().numpy(), O.mlp_gateup_ref(x[rows], trip(gate), trip(up), g), f"gate/up M={m}")
    del Dg, Du, gsw, usw
    # down_proj (long K: 128-column strips from 256 rows on)
    down = O.make_layer(I, H, g, seed=1802)
    Dd = to_dev(down)
    dsw, dm = G.stream_pack(Dd["qweight"], Dd["qzeros"], Dd["scales"], g)
    h = O.make_x(m, I, seed=m + 8)
    hd = torch.from_numpy(h).cuda()
    ys = G.matmul4_stream(g, hd, dsw, dm)
    assert_close(ys[rows].cpu().numpy(), O.quant_matmul_ref(h[rows], *trip(down), g), f"down_proj M={m}")
    del Dd, dsw
    # fused QKV + rotary
    L = O.make_layer(H, 3 * H, g, seed=1803)
    D = to_dev(L)
    sw, meta = G.stream_pack(D["qweight"], D["qzeros"], D["scales"], g)
    pos = (np.arange(m, dtype=np.int64)[None, :] + 5)
    cos, sin = G.RotaryTable(128, 2048).get(torch.device("cuda"), 2048)
    x3 = torch.from_numpy(x.reshape(1, m, H)).cuda()
    q, kk, vv = G.qkv_rotary_stream(g, x3, sw, meta, torch.from_numpy(pos).cuda(), cos, sin, heads)
    q2, k2, v2 = G.qkv_rotary(g, x3, D["qweight"], D["scales"], D["qzeros"], torch.from_numpy(pos).cuda(), cos, sin, heads)
    for a, b in ((q, q2), (kk, k2), (vv, v2)):
        ok, max_abs, _ = O.within_tolerance(a.cpu().numpy(), b.float().cpu().numpy())
        assert ok, max_abs
    qr, kr, vr = O.qkv_rotary_ref(x.reshape(1, m, H)[:, rows], L["qweight"], L["qzeros"], L["scales"], g, pos[:, rows], heads, max_pos=2048)
    for got, ref, name in ((q, qr, "q"), (kk, kr, "k"), (vv, vr, "v")):
        assert_close(got[:, :, rows].cpu().numpy(), ref, f"qkv {name} M={m}")
    assert head_is_zero()


@pytest.mark.parametrize("waves,depth", [(8, 1), (8, 3), (16, 1), (16, 2)])
def test_matmul_in_every_launch_shape(waves, depth):
    G = gptq()
    _lib = lib_()
    lib = _lib.load()
    try:
        lib.gptq4_set_stream_tuning(waves, depth)
        for (k, n, g) in ((2048, 512, 128), (4096, 4096, 128), (11008, 4096, 128)):
            L = O.make_layer(k, n, g, seed=1100 + k)
            D = to_dev(L)
            sw, meta = G.stream_pack(D["qweight"], D["qzeros"], D["scales"], g)
            for m in (1, 4) + ((9, 16) if depth <= 2 else ()):
                x = O.make_x(m, k, seed=m)
                y = G.matmul4_stream(g, torch.from_numpy(x).cuda(), sw, meta)
                assert_close(y.cpu().numpy(), O.quant_matmul_ref(x, L["qweight"], L["qzeros"], L["scales"], g), f"{waves}x{depth} {k}x{n} M={m}")
    finally:
        lib.gptq4_set_stream_tuning(0, 0)
    assert head_is_zero()


@pytest.mark.parametrize("mode", [10, 20])  # 5 .. 16 rows: one tile per unit of loads everywhere / two wherever they can run
def test_rows_5_to_16_with_one_and_with_two_tiles_per_unit(mode):
    G = gptq()
    _lib = lib_()
    lib = _lib.load()
    trip = lambda d: (d["qweight"], d["qzeros"], d["scales"])
    try:
        lib.gptq4_set_stream_tuning(0, mode)
        for m in (5, 8, 13, 16):
            # plain projections, with and without a bias; ranges that cut tiles (2048 x 512: 4 units to a workgroup) and long ones
            for (k, n, g) in ((2048, 512, 128), (4096, 4096, 128), (11008, 4096, 128), (1024, 7168, 256)):
                L = O.make_layer(k, n, g, seed=1700 + k + n, bias=(m == 8))
                D = to_dev(L)
                sw, meta = G.stream_pack(D["qweight"], D["qzeros"], D["scales"], g)
                x = O.make_x(m, k, seed=m + 7)
                y = G.matmul4_stream(g, torch.from_numpy(x).cuda(), sw, meta, D.get("bias"))
                ref = O.quant_matmul_ref(x, *trip(L), g, bias=L.get("bias"))
                if L.get("bias") is None:
                    assert_close(y.cpu().numpy(), ref, f"mode {mode} {k}x{n} M={m}")
                else:  # (two fp16 roundings, as the reference's: the tight bound of assert_close does not apply)
                    ok, max_abs, _ = O.within_tolerance(y.cpu().numpy(), ref)
                    assert ok, f"mode {mode} {k}x{n} M={m} with bias: max_abs={max_abs}"
            for (k, inter, g) in ((1024, 2816, 128), (4096, 11008, 128)):
                gate, up = O.make_layer(k, inter, g, seed=1710 + k), O.make_layer(k, inter, g, seed=1711 + k)
                Dg, Du = to_dev(gate), to_dev(up)
                gsw, gm = G.stream_pack(Dg["qweight"], Dg["qzeros"], Dg["scales"], g)
                usw, um = G.stream_pack(Du["qweight"], Du["qzeros"], Du["scales"], g)
                x = O.make_x(m, k, seed=m + 51)
                y = G.llama_mlp_4_stream(g, torch.from_numpy(x).cuda(), gsw, gm, usw, um)
                assert_close(y.cpu().numpy(), O.mlp_gateup_ref(x, trip(gate), trip(up), g), f"mode {mode} gate/up {k}x{inter} M={m}")
            for (k, heads, g) in ((1024, 8, 128), (4096, 32, 128)):
                L = O.make_layer(k, 3 * heads * 128, g, seed=1720 + k)
                D = to_dev(L)
                sw, meta = G.stream_pack(D["qweight"], D["qzeros"], D["scales"], g)
                x = O.make_x(m, k, seed=m + 61).reshape(m, 1, k)
                pos = (np.arange(m)[:, None] * 29 + 2047 - 29 * (m - 1)).astype(np.int64)
                cos, sin = G.RotaryTable(128, 2048).get(torch.device("cuda"), 2048)
                q, kk, vv = G.qkv_rotary_stream(g, torch.from_numpy(x).cuda(), sw, meta, torch.from_numpy(pos).cuda(), cos, sin, heads)
                refs = O.qkv_rotary_ref(x, *trip(L), g, pos, heads, max_pos=2048)
                for got, ref, name in zip((q, kk, vv), refs, "qkv"):
                    assert_close(got.cpu().numpy(), ref, f"mode {mode} qkv {name} K={k} M={m}")
    finally:
        lib.gptq4_set_stream_tuning(0, 0)
    assert head_is_zero()


def test_one_hot_rows_return_weight_rows_exactly():
    """x = e_k: the result is row k of the dequantised weight, exactly (a single term, no rounding but the weight's own)."""
    G = gptq()
    k, n, g = 4096, 4096, 128
    L = O.make_layer(k, n, g, seed=1200)
    D = to_dev(L)
    sw, meta = G.stream_pack(D["qweight"], D["qzeros"], D["scales"], g)
    w = O.dequant_fp16(L["qweight"], L["qzeros"], L["scales"], g)
    for rows in ([0, 1, 127, 128], [4095, 2049, 3000, 77]):
        x = np.zeros((4, k), dtype=np.float16)
        for i, r in enumerate(rows):
            x[i, r] = 1.0
        y = G.matmul4_stream(g, torch.from_numpy(x).cuda(), sw, meta)
        assert (bits(y.cpu().numpy()) == bits(w[rows])).all()
    # sixteen rows: the kernel that fetches its rows with every unit
    rows = [0, 1, 7, 8, 31, 32, 127, 128, 129, 1000, 2047, 2048, 3000, 4000, 4094, 4095]
    x = np.zeros((16, k), dtype=np.float16)
    for i, r in enumerate(rows):
        x[i, r] = 1.0
    y = G.matmul4_stream(g, torch.from_numpy(x).cuda(), sw, meta)
    assert (bits(y.cpu().numpy()) == bits(w[rows])).all()


@pytest.mark.parametrize("k,n,g", [(1024, 512, 128), (4096, 4096, 128), (5120, 5120, 128)])
@pytest.mark.parametrize("m", [1, 3, 6, 16])
def test_matmul_act_order(k, n, g, m):
    """Rows sorted by group first (gptq4_actorder_sort_rows), then streaming order; x gathered through perm inside the kernel."""
    G = gptq()
    L = O.make_layer(k, n, g, seed=1300 + k, act_order=True)
    D = to_dev(L)
    qs, perm = G.prepare_act_order(D["qweight"], D["g_idx"], g)
    sw, meta = G.stream_pack(qs, D["qzeros"], D["scales"], g)
    x = O.make_x(m, k, seed=m + 40)
    y = G.matmul4_stream(g, torch.from_numpy(x).cuda(), sw, meta, None, perm)
    ref = O.quant_matmul_ref(x, L["qweight"], L["qzeros"], L["scales"], g, g_idx=L["g_idx"])
    assert_close(y.cpu().numpy(), ref, f"act-order stream matmul {k}x{n} M={m}")


@pytest.mark.parametrize("k,inter,g", [(1024, 2816, 128), (4096, 11008, 128), (5120, 13824, 128), (6656, 17920, 512)])
@pytest.mark.parametrize("m", [1, 2, 4, 5, 11, 16])
def test_mlp_gateup(k, inter, g, m):
    G = gptq()
    gate, up = O.make_layer(k, inter, g, seed=1400 + k), O.make_layer(k, inter, g, seed=1401 + k)
    Dg, Du = to_dev(gate), to_dev(up)
    if G.quant_linear.stream_rows(1, k, inter, g) < m:
        pytest.skip("shape outside what the streaming-order kernel takes")
    gsw, gm = G.stream_pack(Dg["qweight"], Dg["qzeros"], Dg["scales"], g)
    usw, um = G.stream_pack(Du["qweight"], Du["qzeros"], Du["scales"], g)
    x = O.make_x(m, k, seed=m + 50)
    y = G.llama_mlp_4_stream(g, torch.from_numpy(x).cuda(), gsw, gm, usw, um)
    trip = lambda d: (d["qweight"], d["qzeros"], d["scales"])
    assert_close(y.cpu().numpy(), O.mlp_gateup_ref(x, trip(gate), trip(up), g), f"stream gate/up {k}x{inter} M={m}")
    assert head_is_zero()


@pytest.mark.parametrize("k,heads,g", [(1024, 8, -1), (4096, 32, -1), (4096, 32, 128), (5120, 40, 128), (6656, 52, 512)])
@pytest.mark.parametrize("m", [1, 4, 7, 16])
def test_qkv_rotary_and_cache_rows(k, heads, g, m):
    G = gptq()
    n = 3 * heads * 128
    gs = k if g == -1 else g
    L = O.make_layer(k, n, g, seed=1500 + k)
    D = to_dev(L)
    if G.quant_linear.stream_rows(2, k, n, gs) < m:
        pytest.skip("shape outside what the streaming-order kernel takes")
    sw, meta = G.stream_pack(D["qweight"], D["qzeros"], D["scales"], gs)
    x = O.make_x(m, k, seed=m + 60).reshape(m, 1, k)
    pos = (np.arange(m)[:, None] * 37 + 2047 - 37 * (m - 1)).astype(np.int64)  # distinct, the last one at the table's end
    cos, sin = G.RotaryTable(128, 2048).get(torch.device("cuda"), 2048)
    xd, posd = torch.from_numpy(x).cuda(), torch.from_numpy(pos).cuda()
    q, kk, vv = G.qkv_rotary_stream(gs, xd, sw, meta, posd, cos, sin, heads)
    qr, kr, vr = O.qkv_rotary_ref(x, L["qweight"], L["qzeros"], L["scales"], g, pos, heads, max_pos=2048)
    for got, ref, name in ((q, qr, "q"), (kk, kr, "k"), (vv, vr, "v")):
        assert_close(got.cpu().numpy(), ref, f"stream qkv {name} K={k} M={m}")
    # straight into a KV cache, at the row of each token's position: only those rows change
    cap = 2048
    kc = torch.full((m, heads, cap, 128), 7.0, dtype=torch.float16, device="cuda")
    vc = torch.full_like(kc, -3.0)
    q2, _, _ = G.qkv_rotary_stream(gs, xd, sw, meta, posd, cos, sin, heads, kv_out=(kc, vc), kv_offset=-1)
    assert torch.equal(q2, q)
    for b in range(m):
        row = int(pos[b, 0])
        assert torch.equal(kc[b, :, row], kk[b, :, 0]) and torch.equal(vc[b, :, row], vv[b, :, 0])
        mask = torch.ones(cap, dtype=torch.bool, device="cuda")
        mask[row] = False
        assert bool((kc[b][:, mask] == 7.0).all()) and bool((vc[b][:, mask] == -3.0).all())
    assert head_is_zero()


# ------------------------------------------------------------------ fused residual add + RMSNorm
def residual_inputs(m, hidden, seed):
    rng = np.random.default_rng(seed)
    h = (rng.standard_normal((m, hidden)) * 2).astype(np.float16)
    d = rng.standard_normal((m, hidden)).astype(np.float16)
    w = (1.0 + 0.1 * rng.standard_normal(hidden)).astype(np.float16)
    return h, d, w


@pytest.mark.parametrize("hidden,heads,inter,g,act", [(1024, 8, 2816, 128, False), (4096, 32, 11008, 128, False), (5120, 40, 13824, 128, True)])
@pytest.mark.parametrize("m", [1, 2, 4])
@pytest.mark.parametrize("with_delta", [True, False])
def test_normalising_variants_equal_norm_launch_plus_plain_call(hidden, heads, inter, g, act, m, with_delta):
    G = gptq()
    from gptq_triton_amd.decoder_ops import add_rms_norm, rms_norm
    qkv = O.make_layer(hidden, 3 * hidden, g, seed=1600, act_order=act)
    gate, up = O.make_layer(hidden, inter, g, seed=1601, act_order=act), O.make_layer(hidden, inter, g, seed=1602)
    Dq, Dg, Du = to_dev(qkv), to_dev(gate), to_dev(up)
    perm = None
    if act:  # one permutation for the projections that share their input
        Dq["qweight"], perm = G.prepare_act_order(Dq["qweight"], Dq["g_idx"], g)
        gate2 = dict(gate, g_idx=qkv["g_idx"])
        Dg["qweight"], _ = G.prepare_act_order(Dg["qweight"], Dq["g_idx"], g)
        Du["qweight"], _ = G.prepare_act_order(Du["qweight"], Dq["g_idx"], g)
    sq, mq = G.stream_pack(Dq["qweight"], Dq["qzeros"], Dq["scales"], g)
    sg, mg = G.stream_pack(Dg["qweight"], Dg["qzeros"], Dg["scales"], g)
    su, mu = G.stream_pack(Du["qweight"], Du["qzeros"], Du["scales"], g)
    h, d, w = residual_inputs(m, hidden, seed=m + 70)
    hd, dd, wd = (torch.from_numpy(t).cuda() for t in (h, d, w))
    hd3 = hd.view(m, 1, hidden)
    eps = 1e-6
    if with_delta:
        s_ref, x_ref = add_rms_norm(hd, dd, wd, eps)
    else:
        s_ref, x_ref = hd, rms_norm(hd, wd, eps)
    pos = torch.arange(m, dtype=torch.int32, device="cuda").view(m, 1) * 5 + 3
    cos, sin = G.RotaryTable(128, 2048).get(torch.device("cuda"), 2048)
    h0, d0 = hd.clone(), dd.clone()
    q0, k0, v0 = G.qkv_rotary_stream(g, x_ref.view(m, 1, hidden), sq, mq, pos, cos, sin, heads, perm=perm)
    q, k, v, s = G.qkv_rotary_stream(g, hd3, sq, mq, pos, cos, sin, heads, perm=perm, norm=(dd.view(m, 1, hidden) if with_delta else None, wd, eps))
    assert torch.equal(q, q0) and torch.equal(k, k0) and torch.equal(v, v0) and torch.equal(s.view(m, hidden), s_ref)
    mid0 = G.llama_mlp_4_stream(g, x_ref, sg, mg, su, mu, perm)
    s2, mid = G.llama_mlp_4_stream(g, hd, sg, mg, su, mu, perm, norm=(dd if with_delta else None, wd, eps))
    assert torch.equal(mid, mid0) and torch.equal(s2, s_ref)
    assert torch.equal(hd, h0) and torch.equal(dd, d0), "inputs must stay untouched"
    assert head_is_zero()


# ------------------------------------------------------------------ the exchange between workgroups
def test_a_wait_that_runs_out_sets_the_error_word_and_the_kernel_still_ends():
    """Spin limit 0xFFFFFFFF, the library's hook for this test: a workgroup that finishes a strip shared with a lower
    one polls once and gives up whatever it found.  The call returns, the error word of its workspace is set.  (A
    private workspace: it is left dirty.)  4096 -> 11008: 688 strips on 256 workgroups, so most range boundaries cut a strip."""
    G = gptq()
    _lib = lib_()
    lib = _lib.load()
    k, n, g, m = 4096, 11008, 128, 1
    L = O.make_layer(k, n, g, seed=1700)
    D = to_dev(L)
    sw, meta = G.stream_pack(D["qweight"], D["qzeros"], D["scales"], g)
    xd = torch.from_numpy(O.make_x(m, k, seed=6)).cuda()
    y = torch.empty((m, n), dtype=torch.float16, device="cuda")
    ws = torch.zeros(_lib.WS_HEAD_BYTES, dtype=torch.uint8, device="cuda")
    stream = _lib.current_stream(xd.device)

    def call():
        return lib.gptq4_stream_matmul(xd.data_ptr(), sw.data_ptr(), meta.data_ptr(), None, None, y.data_ptr(), m, k, n, g,
                                       ws.data_ptr(), ws.numel(), stream)

    def error_word():
        torch.cuda.synchronize()
        return int(ws[4 * _lib.WS_ERROR_WORD:4 * _lib.WS_ERROR_WORD + 4].view(torch.int32).item())

    try:
        assert call() == 0 and error_word() == 0
        assert_close(y.cpu().numpy(), O.quant_matmul_ref(O.make_x(m, k, seed=6), L["qweight"], L["qzeros"], L["scales"], g), "before the limit is lowered")
        lib.gptq4_set_exchange_spin_limit(0xFFFFFFFF)
        assert call() == 0
        assert error_word() == 1
    finally:
        lib.gptq4_set_exchange_spin_limit(0)


def test_host_side_argument_errors():
    _lib = lib_()
    lib = _lib.load()
    fake, ws = 0x1000, _lib.WS_HEAD_BYTES
    assert lib.gptq4_stream_matmul(None, fake, fake, None, None, fake, 1, 4096, 4096, 128, fake, ws, None) == -1
    assert lib.gptq4_stream_matmul(fake, fake, fake, fake, None, fake, 5, 4096, 4096, 128, fake, ws, None) == -4     # act-order above four rows: room for the gathered rows
    assert lib.gptq4_stream_mlp_gateup(fake, None, fake, 1e-6, None, fake, fake, fake, fake, None, fake, 5, 4096, 11008, 128, fake, ws, None) == -2  # norm inside: four rows
    assert lib.gptq4_stream_matmul(fake, fake, fake, None, None, fake, 1, 512, 4096, 128, fake, ws, None) == -2      # K too short for its waves
    assert lib.gptq4_stream_matmul(fake, fake, fake, None, None, fake, 1, 4096, 4096, 96, fake, ws, None) == -3
    assert lib.gptq4_stream_matmul(fake, fake, fake, None, None, fake, 1, 4096, 4096, 128, fake, 64, None) == -4
    assert lib.gptq4_stream_matmul(fake + 2, fake, fake, None, None, fake, 1, 4096, 4096, 128, fake, ws, None) == -5
    assert lib.gptq4_stream_rows(0, 4096, 4096, 128) == 16 and lib.gptq4_stream_rows(0, 512, 4096, 128) == 0
    assert lib.gptq4_stream_rows(0, 4096, 4100, 128) == 0


# ------------------------------------------------------------------ the modules
def _quant_linear(k, n, g, seed, act, bias=False):
    G = gptq()
    L = O.make_layer(k, n, g, seed=seed, act_order=act, bias=bias)
    q = G.QuantLinear(4, g, k, n, bias, act_order=act)
    q.qweight.copy_(torch.from_numpy(L["qweight"]))
    q.qzeros.copy_(torch.from_numpy(L["qzeros"]))
    q.scales.copy_(torch.from_numpy(L["scales"]))
    if bias:
        q.bias.copy_(torch.from_numpy(L["bias"]))
    if act:
        q.g_idx.copy_(torch.from_numpy(L["g_idx"]))
    return q, L


@pytest.mark.parametrize("act", [False, True])
def test_quant_linear_in_streaming_order(act):
    """to_stream(): same results (oracle), ONE copy of the weight, state_dict / dequantize / checkpoint_qweight still in the
    checkpoint layout - on the GPU and after the module has been moved to the CPU - and load_state_dict brings it back."""
    G = gptq()
    k, n, g = 4096, 4096, 128
    q, L = _quant_linear(k, n, g, 1800, act, bias=True)
    q = q.cuda()
    before = {name: t.clone() for name, t in q.state_dict().items()}
    w_before = q.dequantize()
    assert q.to_stream() and q._stream_rows == 16
    assert q.qweight.shape == before["qweight"].shape and not torch.equal(q.qweight, before["qweight"])
    for m in (1, 4, 9, 16, 33):   # 33 rows: unpacked for the duration of the call, tiled kernels
        x = O.make_x(m, k, seed=m)
        y = q(torch.from_numpy(x).cuda())
        ref = O.quant_matmul_ref(x, L["qweight"], L["qzeros"], L["scales"], g, bias=L["bias"], g_idx=L["g_idx"] if act else None)
        ok, max_abs, _ = O.within_tolerance(y.cpu().numpy(), ref)   # (fp16(acc) + fp16 bias: two roundings, so no tighter bound here)
        assert ok, f"QuantLinear in streaming order, act-order {act}, M={m}: {max_abs}"
    after = q.state_dict()
    assert set(after) == set(before) and all(torch.equal(after[name], before[name]) for name in before)
    assert torch.equal(q.dequantize(), w_before) and torch.equal(q.checkpoint_qweight(), before["qweight"])
    cpu_state = q.cpu().state_dict()
    assert all(torch.equal(cpu_state[name], before[name].cpu()) for name in before)
    q = q.cuda()
    q.load_state_dict(before)
    assert q._stream_meta is None and q._compact_perm is None and torch.equal(q.qweight, before["qweight"])
    q.to_stream()
    q.to_checkpoint()
    assert q._stream_meta is None and torch.equal(q.checkpoint_qweight(), before["qweight"])


@pytest.mark.parametrize("act", [False, True])
def test_fused_mlp_in_streaming_order(act):
    G = gptq()
    k, inter, g = 1024, 2816, 128
    gate, Lg = _quant_linear(k, inter, g, 1900, act)
    up, Lu = _quant_linear(k, inter, g, 1901, act)
    down, Ld = _quant_linear(inter, k, g, 1902, act)
    if act:
        up.g_idx.copy_(gate.g_idx)
        Lu["g_idx"] = Lg["g_idx"]
    mlp = G.QuantLlamaMLP(gate, down, up).cuda()
    before = {name: t.clone() for name, t in mlp.state_dict().items()}
    x = O.make_x(3, k, seed=5)
    xd = torch.from_numpy(x).cuda()
    y_ckpt = mlp(xd)
    x12 = torch.from_numpy(O.make_x(12, k, seed=7)).cuda()
    y12_ckpt = mlp(x12)
    assert mlp.to_stream() and mlp.down_proj._stream_meta is not None
    y = mlp(xd)
    # twelve rows: the streaming-order kernel for 5 .. 16 rows (an act-order block's rows are gathered by a launch before it)
    ok, max_abs, _ = O.within_tolerance(mlp(x12).float().cpu().numpy(), y12_ckpt.float().cpu().numpy())
    assert ok, max_abs
    # same fp16 intermediate up to the order of the fp32 sums: compare both against the oracle's composed result
    trip = lambda d: (d["qweight"], d["qzeros"], d["scales"])
    if not act:
        mid = O.mlp_gateup_ref(x, trip(Lg), trip(Lu), g).astype(np.float16)
        ref = O.quant_matmul_ref(mid, *trip(Ld), g)
        ok, max_abs, _ = O.within_tolerance(y.cpu().numpy(), ref)
        assert ok, max_abs
    ok, max_abs, _ = O.within_tolerance(y.cpu().numpy(), y_ckpt.float().cpu().numpy())
    assert ok, max_abs
    y33 = mlp(torch.from_numpy(O.make_x(33, k, seed=6)).cuda())   # tall call on the streamed block
    assert y33.shape == (33, k) and bool(torch.isfinite(y33).all())
    after = mlp.state_dict()
    assert set(after) == set(before) and all(torch.equal(after[name], before[name]) for name in before)
    cpu_state = mlp.cpu().state_dict()
    assert all(torch.equal(cpu_state[name], before[name].cpu()) for name in before)
    mlp = mlp.cuda()
    mlp.load_state_dict(before)
    assert mlp._gate_meta is None and torch.equal(mlp.gate_proj_qweight, before["gate_proj_qweight"])


def random_quant_model(hidden, inter, heads, layers, groupsize, seed, act_order=False):
    """A random-init decoder of the given shape on the GPU, attention and MLP blocks fused."""
    G = gptq()
    from gptq_triton_amd.llama import LlamaForCausalLM, LlamaRMSNorm
    cfg = G.LlamaConfigLite(hidden_size=hidden, num_attention_heads=heads, max_position_embeddings=512, intermediate_size=inter,
                            num_hidden_layers=layers, vocab_size=320)
    dev = torch.device("cuda")
    gen = torch.Generator(device=dev).manual_seed(seed)
    model = LlamaForCausalLM(cfg).half()
    G.make_quant(model, 4, groupsize, act_order=act_order)
    model = model.to(dev)
    for layer in model.model.layers:
        perms = {}
        for group, names in (("attn_in", ("self_attn.q_proj", "self_attn.k_proj", "self_attn.v_proj")), ("attn_out", ("self_attn.o_proj",)),
                             ("mlp_in", ("mlp.gate_proj", "mlp.up_proj")), ("mlp_out", ("mlp.down_proj",))):
            for name in names:
                q = layer.get_submodule(name)
                q.qweight.copy_(torch.randint(-2**31, 2**31 - 1, q.qweight.shape, dtype=torch.int32, device=dev, generator=gen))
                q.qzeros.copy_(torch.randint(-2**31, 2**31 - 1, q.qzeros.shape, dtype=torch.int32, device=dev, generator=gen))
                q.scales.copy_(((0.2 + 0.3 * torch.rand(q.scales.shape, device=dev, generator=gen)) / (4.6 * q.infeatures ** 0.5)).half())
                if act_order:
                    if group not in perms:
                        base = torch.arange(q.infeatures, device=dev) // groupsize
                        perms[group] = base[torch.randperm(q.infeatures, device=dev, generator=gen)].int()
                    q.g_idx.copy_(perms[group])
    with torch.no_grad():
        for m in model.modules():
            if isinstance(m, LlamaRMSNorm):
                m.weight.fill_(1.0)
        model.model.embed_tokens.weight.copy_(torch.randn(model.model.embed_tokens.weight.shape, device=dev, generator=gen) * 0.5)
        model.lm_head.weight.copy_(torch.randn(model.lm_head.weight.shape, device=dev, generator=gen) * 0.02)
    G.make_quant_attn(model)
    G.make_fused_mlp(model)
    return model


@pytest.mark.parametrize("act_order", [False, True])
def test_greedy_decoder_in_streaming_order_matches_the_checkpoint_layout(act_order):
    """A small random decoder: the same greedy tokens from the streaming-order layout (one sequence and three: the kernel
    with the rows in LDS, the norms fused into the projections; six: the kernel that fetches the rows with every unit; twenty:
    the mid-M kernel on the same words) as from the checkpoint layout, eager and as a replayed graph."""
    G = gptq()
    model = random_quant_model(hidden=1024, inter=2816, heads=8, layers=2, groupsize=128, seed=7, act_order=act_order)
    for bsz in (1, 3, 6, 20):
        ids = torch.randint(0, model.config.vocab_size, (bsz, 12), device="cuda", generator=torch.Generator(device="cuda").manual_seed(bsz))
        G.set_layout(model, "checkpoint")
        dec = G.GreedyDecoder(model, bsz, 64, layout="keep")
        first = dec.prefill(ids)
        want = torch.cat([first, dec.decode(10)], dim=1)
        dec = G.GreedyDecoder(model, bsz, 64)   # 'auto': streaming order
        assert model.model.layers[0].self_attn.qkv_proj._stream_meta is not None
        first = dec.prefill(ids)
        got = torch.cat([first, dec.decode(10, use_graph=True)], dim=1)
        if bsz <= 4:
            assert torch.equal(got, want), (bsz, got.tolist(), want.tolist())
        else:
            # other kernels on both sides, other orders of the fp32 sums: a near-tie between two logits may go the other way
            # (and the sequence then continues differently); most sequences agree to the last token
            same = (got == want).all(dim=1).float().mean().item()
            assert same >= 0.8 and torch.equal(got[:, 0], want[:, 0]) or same >= 0.9, (bsz, same)
    G.set_layout(model, "checkpoint")
