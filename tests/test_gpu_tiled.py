"""GPU parity of the tiled kernel with the mid-M kernel switched off, so that every row count
above 16 reaches it: both workgroup tiles (128 x 128 and 128 x 256), with and without K split
across workgroups, all three epilogues, ragged last row tiles, and the automatic plan on a
shape with enough wide tiles.  Same bars as test_gpu_parity.py."""
import numpy as np
import pytest
import torch

from conftest import to_dev
from oracle import gptq_oracle as O
from test_gpu_parity import assert_close, gptq

pytestmark = pytest.mark.gpu

# (32-row blocks per wave: 2 = 128 x 128 tile, 4 = 128 x 256 tile; split-K); 0 = automatic; 200 = the streamed
# schedule (K tiles of all wide tiles dealt evenly to 512 workgroups: at these sizes one K tile each and up to
# 64 sharers per tile), 100 = never streamed
CONFIGS = [(2, 1), (4, 1), (2, 3), (4, 2), (0, 0), (200, 0), (100, 0)]


@pytest.fixture(params=CONFIGS, ids=lambda c: "mt%d_s%d" % c)
def forced_tiled(request):
    from gptq_triton_amd import _lib
    lib = _lib.load()
    lib.gptq4_set_midm_tuning(0, 0, 0)
    lib.gptq4_set_gemm_tuning(*request.param)
    yield lib
    lib.gptq4_set_gemm_tuning(0, 0)
    lib.gptq4_set_midm_tuning(1, 0, 0)


@pytest.mark.parametrize("k,n,g", [(1024, 512, 128), (1536, 256, -1), (2048, 768, 512)])
@pytest.mark.parametrize("m", [17, 128, 130, 300])
def test_tiled_matmul(forced_tiled, k, n, g, m):
    L = O.make_layer(k, n, g, seed=k + n + m, bias=(m % 2 == 0))
    x = O.make_x(m, k, seed=m + 5)
    D = to_dev(L)
    xd = torch.from_numpy(x).cuda()
    y = gptq().matmul4(k if g == -1 else g, xd, D["qweight"], D["scales"], D["qzeros"], D.get("bias"))
    y2 = gptq().matmul4(k if g == -1 else g, xd, D["qweight"], D["scales"], D["qzeros"], D.get("bias"))
    assert torch.equal(y, y2)
    ref = O.quant_matmul_ref(x, L["qweight"], L["qzeros"], L["scales"], g, bias=L["bias"])
    if L["bias"] is None:
        assert_close(y.cpu().numpy(), ref, f"tiled matmul K={k} N={n} g={g} M={m}")
    else:
        ok, max_abs, _ = O.within_tolerance(y.cpu().numpy(), ref)
        assert ok, max_abs


@pytest.mark.parametrize("m", [40, 200])
def test_tiled_gateup(forced_tiled, m):
    k, n, g = 1024, 1280, 128
    gate = O.make_layer(k, n, g, seed=100)
    up = O.make_layer(k, n, g, seed=101)
    x = O.make_x(m, k, seed=102 + m)
    Dg, Du = to_dev(gate), to_dev(up)
    h = gptq().llama_mlp_4(g, torch.from_numpy(x).cuda(), Dg["qweight"], Dg["scales"], Dg["qzeros"],
                           Du["qweight"], Du["scales"], Du["qzeros"])
    ref = O.mlp_gateup_ref(x, (gate["qweight"], gate["qzeros"], gate["scales"]),
                           (up["qweight"], up["qzeros"], up["scales"]), g)
    assert_close(h.cpu().numpy(), ref, f"tiled gate/up M={m}")


@pytest.mark.parametrize("b,s,pos0,g", [(2, 33, 10, 128), (40, 1, 500, -1), (1, 150, 1800, 128)])
def test_tiled_qkv_rotary(forced_tiled, b, s, pos0, g):
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
        assert_close(got.cpu().numpy(), ref, f"tiled {name} b={b} s={s} g={g}")


def test_tiled_rotary_by_position_with_positions_outside_the_table(forced_tiled):
    """Cache rows placed by position id (kv_offset = KV_AT_POSITION) in the tiled kernel, with position ids below 0
    and past the end of the cos / sin tables: the angle is that of the nearest table row, the cache row is the
    position clamped into the cache.  150 tokens per sequence: a ragged last row tile."""
    from gptq_triton_amd.fused_attention import KV_AT_POSITION
    H, Dh, hidden, g = 8, 128, 1024, 128
    L = O.make_layer(hidden, 3 * hidden, g, seed=520)
    D = to_dev(L)
    G = gptq()
    max_pos, cap, b, s = 96, 256, 2, 150
    cos, sin = G.RotaryTable(Dh, max_pos).get(torch.device("cuda"), max_pos)
    cos, sin = cos[:max_pos].contiguous(), sin[:max_pos].contiguous()
    rng = np.random.default_rng(521)
    pos = np.stack([1 + rng.permutation(cap - 1)[:s] for _ in range(b)]).astype(np.int64)   # distinct cache rows, none 0
    pos[0, 7], pos[1, 140] = -3, -1                                                          # these go to row 0
    x = O.make_x(b * s, hidden, seed=522).reshape(b, s, hidden)
    kc = torch.full((b, H, cap, Dh), 7.0, dtype=torch.float16, device="cuda")
    vc = torch.full((b, H, cap, Dh), 7.0, dtype=torch.float16, device="cuda")
    xd, pd = torch.from_numpy(x).cuda(), torch.from_numpy(pos).cuda()
    q, _, _ = G.qkv_rotary(g, xd, D["qweight"], D["scales"], D["qzeros"], pd, cos, sin, H, Dh,
                           kv_out=(kc, vc), kv_offset=KV_AT_POSITION)
    angle_row = np.clip(pos, 0, max_pos - 1)
    qr, kr, vr = O.qkv_rotary_ref(x, L["qweight"], L["qzeros"], L["scales"], g, angle_row, H, Dh, max_pos=max_pos)
    assert_close(q.cpu().numpy(), qr, "q by position")
    cache_row = np.clip(pos, 0, cap - 1)
    for bi in range(b):
        rows = torch.from_numpy(cache_row[bi]).cuda()
        assert_close(kc[bi][:, rows].cpu().numpy(), kr[bi], f"k rows of sequence {bi}")
        assert_close(vc[bi][:, rows].cpu().numpy(), vr[bi], f"v rows of sequence {bi}")
        untouched = torch.ones(cap, dtype=torch.bool)
        untouched[cache_row[bi]] = False
        assert bool((kc[bi][:, untouched] == 7.0).all()) and bool((vc[bi][:, untouched] == 7.0).all())


@pytest.mark.parametrize("m", [1100, 2048])
def test_streamed_schedule_at_prefill_size(m):
    """The streamed schedule on a tile count that does not divide by the resident workgroups (1100 rows x 8192
    columns = 9 x 32 wide tiles, the last row tile ragged; 2048 x 8192 = 512 tiles, one each): every workgroup gets
    the same number of K tiles, tiles cut by a range boundary are finished by whoever arrives last.  Against the
    oracle on sampled rows and the tile-boundary rows, and against the unstreamed schedule within rounding (the
    partial sums meet in another order); two calls give the same bits."""
    from gptq_triton_amd import _lib
    lib = _lib.load()
    G = gptq()
    k, n, g, heads = 2048, 8192, 128, 16
    L = O.make_layer(k, n, g, seed=700, bias=True)
    up = O.make_layer(k, n, g, seed=701)
    qkv = O.make_layer(k, 3 * k, g, seed=702)
    x = O.make_x(m, k, seed=703)
    xd = torch.from_numpy(x).cuda()
    D, Du, Dq = to_dev(L), to_dev(up), to_dev(qkv)
    cos, sin = G.RotaryTable(128, 4096).get(torch.device("cuda"), 4096)
    pos = np.arange(m, dtype=np.int32)[None, :]
    pd = torch.from_numpy(pos).cuda()
    out = {}
    lib.gptq4_set_midm_tuning(0, 0, 0)
    try:
        for mode in (200, 100):
            lib.gptq4_set_gemm_tuning(mode, 0)
            y = G.matmul4(g, xd, D["qweight"], D["scales"], D["qzeros"], D["bias"])
            y2 = G.matmul4(g, xd, D["qweight"], D["scales"], D["qzeros"], D["bias"])
            assert torch.equal(y, y2)
            h = G.llama_mlp_4(g, xd, D["qweight"], D["scales"], D["qzeros"], Du["qweight"], Du["scales"], Du["qzeros"])
            q, kk, vv = G.qkv_rotary(g, xd.view(1, m, k), Dq["qweight"], Dq["scales"], Dq["qzeros"], pd, cos, sin, heads)
            out[mode] = (y, h, q, kk, vv)
    finally:
        lib.gptq4_set_gemm_tuning(0, 0)
        lib.gptq4_set_midm_tuning(1, 0, 0)
    for a, b, name in zip(out[200], out[100], ("matmul", "gate/up", "q", "k", "v")):
        a, b = a.float(), b.float()
        assert bool(((a - b).abs() <= 2e-3 + 2e-3 * b.abs()).all()), f"{name}: streamed and unstreamed schedules differ beyond rounding"
    rows = sorted(set([0, 1, 127, 128, 129, 1023, 1024, m - 129, m - 1] + list(np.random.default_rng(5).integers(0, m, 24))))
    xs = x[rows]
    y, h, q, kk, vv = out[200]
    assert_close_bias = O.within_tolerance(y[rows].cpu().numpy(), O.quant_matmul_ref(xs, L["qweight"], L["qzeros"], L["scales"], g, bias=L["bias"]))
    assert assert_close_bias[0], assert_close_bias[1]
    href = O.mlp_gateup_ref(xs, (L["qweight"], L["qzeros"], L["scales"]), (up["qweight"], up["qzeros"], up["scales"]), g)
    assert_close(h[rows].cpu().numpy(), href, f"streamed gate/up M={m}")
    qr, kr, vr = O.qkv_rotary_ref(xs.reshape(1, len(rows), k), qkv["qweight"], qkv["qzeros"], qkv["scales"], g, pos[:, rows], heads, 128,
                                  max_pos=4096)
    for got, want, name in ((q, qr, "q"), (kk, kr, "k"), (vv, vr, "v")):
        assert_close(got[:, :, rows].cpu().numpy(), want, f"streamed {name} M={m}")


def _parts(lib, op, m, k, n):
    import ctypes
    begin, cols = (ctypes.c_int * 2)(), (ctypes.c_int * 2)()
    count = lib.gptq4_column_parts(op, m, k, n, begin, cols)
    return [(begin[i], cols[i]) for i in range(count)]


def test_tile_counts_just_above_a_whole_number_of_rounds():
    """Wide tiles are dealt one per CU and round.  384 rows x 11008 gate/up columns = 3 x 86 = 258 tiles, two more than
    one round of the 256 CUs: the two are cut along K into parts that run beside the whole tiles.  768 rows = 516
    tiles and 1408 rows of a 32-head QKV = 11 x 48 = 528, four and sixteen more than two rounds: the call runs as two
    launches over column ranges, the columns of the full rounds as wide tiles and the rest planned by itself.  Either
    way the whole tiles have the bits of the plain schedule and every column meets the oracle on sampled rows."""
    from gptq_triton_amd import _lib
    lib = _lib.load()
    G = gptq()
    dev = torch.device("cuda")
    cus = torch.cuda.get_device_properties(dev).multi_processor_count
    if cus != 256:
        pytest.skip("the shapes are chosen for 256 CUs")
    k, n, g = 2048, 11008, 128
    gate, up = O.make_layer(k, n, g, seed=800), O.make_layer(k, n, g, seed=801)
    Dg, Du = to_dev(gate), to_dev(up)
    for m, want_parts in ((384, [(0, n)]), (768, [(0, 85 * 128), (85 * 128, 128)])):
        assert _parts(lib, _lib.OP_MLP_GATEUP, m, k, n) == want_parts
        x = O.make_x(m, k, seed=802 + m)
        xd = torch.from_numpy(x).cuda()
        out = {}
        try:
            for mode in (0, 500):
                lib.gptq4_set_gemm_tuning(mode, 0)
                h = G.llama_mlp_4(g, xd, Dg["qweight"], Dg["scales"], Dg["qzeros"], Du["qweight"], Du["scales"], Du["qzeros"])
                h2 = G.llama_mlp_4(g, xd, Dg["qweight"], Dg["scales"], Dg["qzeros"], Du["qweight"], Du["scales"], Du["qzeros"])
                assert torch.equal(h, h2)
                out[mode] = h
        finally:
            lib.gptq4_set_gemm_tuning(0, 0)
        same = (out[0] == out[500]).float().mean().item()
        assert same > 0.97, f"M={m}: only {same:.3f} of the values have the bits of the plain schedule"
        assert bool(((out[0].float() - out[500].float()).abs() <= 2e-3 + 2e-3 * out[500].float().abs()).all())
        rows = sorted(set([0, 127, 128, 255, 256, m - 1] + list(np.random.default_rng(6).integers(0, m, 20))))
        href = O.mlp_gateup_ref(x[rows], (gate["qweight"], gate["qzeros"], gate["scales"]), (up["qweight"], up["qzeros"], up["scales"]), g)
        assert_close(out[0][rows].cpu().numpy(), href, f"gate/up M={m}")
    # QKV + rotary: 32 heads
    heads, m = 32, 1408
    k = heads * 128
    parts = _parts(lib, _lib.OP_QKV_ROTARY, m, k, 3 * k)
    assert parts == [(0, 46 * 256), (46 * 256, 2 * 256)], parts
    qkv = O.make_layer(k, 3 * k, g, seed=803)
    x = O.make_x(m, k, seed=804)
    xd = torch.from_numpy(x).cuda().view(1, m, k)
    Dq = to_dev(qkv)
    cos, sin = G.RotaryTable(128, 2048).get(dev, 2048)
    pos = np.arange(m, dtype=np.int32)[None, :]
    g = 128
    q, kk, vv = G.qkv_rotary(g, xd, Dq["qweight"], Dq["scales"], Dq["qzeros"], torch.from_numpy(pos).cuda(), cos, sin, heads)
    rows = sorted(set([0, 127, 128, m - 1] + list(np.random.default_rng(7).integers(0, m, 12))))
    qr, kr, vr = O.qkv_rotary_ref(x[rows].reshape(1, len(rows), k), qkv["qweight"], qkv["qzeros"], qkv["scales"], g, pos[:, rows], heads, 128,
                                  max_pos=2048)
    for got, want, name in ((q, qr, "q"), (kk, kr, "k"), (vv, vr, "v")):
        assert_close(got[:, :, rows].cpu().numpy(), want, f"{name} in two launches")


def test_prefill_sized_call_takes_the_wide_tiles_by_itself():
    """2048 rows x 3072 columns = 192 wide tiles: the automatic plan picks the 128 x 256 tile
    without any forcing; K is small so that the oracle finishes in seconds."""
    k, n, g, m = 256, 3072, 128, 2048
    L = O.make_layer(k, n, g, seed=77)
    x = O.make_x(m, k, seed=78)
    D = to_dev(L)
    y = gptq().matmul4(g, torch.from_numpy(x).cuda(), D["qweight"], D["scales"], D["qzeros"])
    ref = O.quant_matmul_ref(x, L["qweight"], L["qzeros"], L["scales"], g)
    assert_close(y.cpu().numpy(), ref, "prefill-sized matmul")


def test_hand_over_between_the_mid_m_and_the_tiled_kernel():
    """768 rows is the last row count the mid-M kernel takes on a narrow layer, 769 the first
    for the tiled kernel: both sides of the boundary against the oracle, and the rows they
    share against each other within fp32 summation-order noise."""
    k, n, g = 512, 512, 128
    L = O.make_layer(k, n, g, seed=91)
    x = O.make_x(769, k, seed=92)
    D = to_dev(L)
    ref = O.quant_matmul_ref(x, L["qweight"], L["qzeros"], L["scales"], g)
    ya = gptq().matmul4(g, torch.from_numpy(x[:768].copy()).cuda(), D["qweight"], D["scales"], D["qzeros"])
    yb = gptq().matmul4(g, torch.from_numpy(x).cuda(), D["qweight"], D["scales"], D["qzeros"])
    assert_close(ya.cpu().numpy(), ref[:768], "768 rows")
    assert_close(yb.cpu().numpy(), ref, "769 rows")
    big = torch.maximum(ya.abs(), yb[:768].abs()).float().cpu().numpy().astype(np.float16)
    ulp = torch.from_numpy(np.spacing(big).astype(np.float32)).cuda()
    assert bool(((ya.float() - yb[:768].float()).abs() <= ulp + 1e-4).all())


def test_tiled_one_hot_rows_reproduce_weight_rows(forced_tiled):
    """x = e_k picks row k of the dequantised weight: a single product, so the tiled kernel's own
    in-register decode (natural k order) must give the canonical fp16 weight bit for bit, for
    every nibble position and both column halves of a word pair."""
    k, n, g = 1024, 512, 128
    L = O.make_layer(k, n, g, seed=19)
    D = to_dev(L)
    rows = np.array(list(range(0, 16)) + [63, 64, 127, 128, 255, 256, 511, 512, 700, 767, 768, 1000, 1016, 1017, 1022, 1023]
                    + list(range(320, 328)))
    x = np.zeros((len(rows), k), dtype=np.float16)
    x[np.arange(len(rows)), rows] = 1.0
    y = gptq().matmul4(g, torch.from_numpy(x).cuda(), D["qweight"], D["scales"], D["qzeros"])
    W = O.dequant_fp16(L["qweight"], L["qzeros"], L["scales"], g)
    assert (y.cpu().numpy().view(np.uint16) == W[rows].view(np.uint16)).all()


@pytest.mark.parametrize("m", [64, 300, 1100])
def test_graph_replays_equal_eager_launches(m):
    """The K-sliced and tiled kernels under HIP-graph capture (split-K counters included): every replay,
    with new input values and eager launches in between, gives the bits of an eager call."""
    k, n, g = 2048, 1024, 128
    L, L2 = O.make_layer(k, n, g, seed=70), O.make_layer(k, n, g, seed=71)
    D, D2 = to_dev(L), to_dev(L2)
    G = gptq()
    x = torch.from_numpy(O.make_x(m, k, seed=72)).cuda()

    def ops():
        return (G.matmul4(g, x, D["qweight"], D["scales"], D["qzeros"]),
                G.llama_mlp_4(g, x, D["qweight"], D["scales"], D["qzeros"], D2["qweight"], D2["scales"], D2["qzeros"]))

    s = torch.cuda.Stream()
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s):
        ops()                                   # sizes this stream's workspace outside the capture
    torch.cuda.current_stream().wait_stream(s)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=s):
        y, h = ops()
    for i in range(4):
        x.copy_(torch.from_numpy(O.make_x(m, k, seed=80 + i)).cuda())
        graph.replay()
        torch.cuda.synchronize()
        y_e, h_e = ops()
        assert torch.equal(y, y_e) and torch.equal(h, h_e), f"replay {i}"
    ref = O.quant_matmul_ref(x.cpu().numpy(), L["qweight"], L["qzeros"], L["scales"], g)
    ok, max_abs, _ = O.within_tolerance(y.cpu().numpy(), ref)
    assert ok, max_abs


@pytest.mark.parametrize("mt", [2, 4])
@pytest.mark.parametrize("m", [40, 200])
def test_in_kernel_act_order_gather_with_fused_epilogues(m, mt):
    """Act-order calls normally run on a gathered copy of the activations; with the tile selector + 10 the tiled
    kernel gathers them itself (what a call does whose copy would pass the staging limit) - also under the
    SiLU*mul and the rotary epilogue."""
    from gptq_triton_amd import _lib
    G = gptq()
    lib = _lib.load()
    k, n, g, heads = 1024, 768, 128, 8
    gate = O.make_layer(k, n, g, seed=90, act_order=True)
    up = O.make_layer(k, n, g, seed=91)
    up["g_idx"] = gate["g_idx"]
    qkv = O.make_layer(k, 3 * k, g, seed=92, act_order=True)
    x = O.make_x(m, k, seed=93)
    xd = torch.from_numpy(x).cuda()
    Dg, Du, Dq = to_dev(gate), to_dev(up), to_dev(qkv)
    gq, perm = G.prepare_act_order(Dg["qweight"], Dg["g_idx"], g)
    uq, _ = G.prepare_act_order(Du["qweight"], Dg["g_idx"], g)
    qq, qperm = G.prepare_act_order(Dq["qweight"], Dq["g_idx"], g)
    stream = _lib.current_stream(xd.device)
    h = torch.empty((m, n), dtype=torch.float16, device="cuda")
    y = torch.empty((m, n), dtype=torch.float16, device="cuda")
    lib.gptq4_set_midm_tuning(0, 0, 0)
    lib.gptq4_set_gemm_tuning(10 + mt, 0)
    ws = _lib.workspace(xd.device, max(lib.gptq4_workspace_bytes(_lib.OP_MLP_GATEUP, m, k, n),
                                       lib.gptq4_workspace_bytes(_lib.OP_QKV_ROTARY, m, k, 3 * k)))
    try:
        _gather_calls(lib, _lib, G, xd, x, m, k, n, g, heads, gate, up, qkv, Dg, Du, Dq, gq, uq, qq, perm, qperm, h, y, ws, stream)
    finally:
        lib.gptq4_set_gemm_tuning(0, 0)
        lib.gptq4_set_midm_tuning(1, 0, 0)


def _gather_calls(lib, _lib, G, xd, x, m, k, n, g, heads, gate, up, qkv, Dg, Du, Dq, gq, uq, qq, perm, qperm, h, y, ws, stream):
    rc = lib.gptq4_matmul(xd.data_ptr(), gq.data_ptr(), Dg["qzeros"].data_ptr(), Dg["scales"].data_ptr(), perm.data_ptr(), None,
                          y.data_ptr(), m, k, n, g, ws.data_ptr(), ws.numel(), stream)
    assert rc == 0
    yref = O.quant_matmul_ref(x, gate["qweight"], gate["qzeros"], gate["scales"], g, g_idx=gate["g_idx"])
    assert_close(y.cpu().numpy(), yref, f"in-kernel gather, matmul M={m}")
    rc = lib.gptq4_mlp_gateup(xd.data_ptr(), gq.data_ptr(), Dg["qzeros"].data_ptr(), Dg["scales"].data_ptr(),
                              uq.data_ptr(), Du["qzeros"].data_ptr(), Du["scales"].data_ptr(), perm.data_ptr(),
                              h.data_ptr(), m, k, n, g, ws.data_ptr(), ws.numel(), stream)
    assert rc == 0
    href = O.mlp_gateup_ref(x, (gate["qweight"], gate["qzeros"], gate["scales"], gate["g_idx"]),
                            (up["qweight"], up["qzeros"], up["scales"], up["g_idx"]), g)
    assert_close(h.cpu().numpy(), href, f"in-kernel gather, gate/up M={m}")
    cos, sin = G.RotaryTable(128, 2048).get(torch.device("cuda"), 2048)
    pos = np.arange(m, dtype=np.int32)[None, :]
    pd = torch.from_numpy(pos).cuda()
    q = torch.empty((1, heads, m, 128), dtype=torch.float16, device="cuda")
    kk, vv = torch.empty_like(q), torch.empty_like(q)
    rc = lib.gptq4_qkv_rotary(xd.data_ptr(), qq.data_ptr(), Dq["qzeros"].data_ptr(), Dq["scales"].data_ptr(), qperm.data_ptr(),
                              pd.data_ptr(), cos.data_ptr(), sin.data_ptr(), cos.shape[0], q.data_ptr(), kk.data_ptr(),
                              vv.data_ptr(), 1, m, heads, 128, k, g, m, 0, ws.data_ptr(), ws.numel(), stream)
    assert rc == 0
    qr, kr, vr = O.qkv_rotary_ref(x.reshape(1, m, k), qkv["qweight"], qkv["qzeros"], qkv["scales"], g, pos, heads, 128,
                                  g_idx=qkv["g_idx"], max_pos=2048)
    for got, want, name in ((q, qr, "q"), (kk, kr, "k"), (vv, vr, "v")):
        assert_close(got.cpu().numpy(), want, f"in-kernel gather, {name} M={m}")
