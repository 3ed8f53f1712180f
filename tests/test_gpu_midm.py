"""GPU parity of the mid-M kernel (K split across the waves of a workgroup), forced on for
every shape it accepts: row counts around its 32- and 64-row tiles and well past them, all
three epilogues, bias, K split across workgroups as well, ragged last row tiles.
Same bars as test_gpu_parity.py."""
import numpy as np
import pytest
import torch

from conftest import to_dev
from oracle import gptq_oracle as O
from test_gpu_parity import assert_close, gptq

pytestmark = pytest.mark.gpu

# (32-row blocks per row tile, split-K across workgroups); 0 = automatic; + 10: 128-column strips for plain
# projections; + 100: four waves per workgroup, + 200: eight (where they fit: 64-row tiles, and 32-row tiles with two
# column blocks per wave tile, only in launches of at most one workgroup per CU); automatic: eight for plain projections
# and, up to 32 rows, for the fused epilogues; + 1000: the rotary epilogue on tiles of 32 columns of a head plus their 32
# rotation partners (automatic: up to 64 rows), + 2000: never
CONFIGS = [(0, 0), (1, 1), (2, 1), (1, 2), (2, 3), (10, 0), (11, 1), (12, 3),
           (100, 0), (101, 1), (102, 1), (101, 3), (102, 2), (111, 2), (112, 1),
           (200, 0), (201, 1), (202, 1), (201, 2), (202, 2), (211, 1), (212, 1),
           (1000, 0), (1001, 1), (1002, 2), (1101, 2), (1102, 1), (1201, 1), (1202, 1), (2000, 0)]

@pytest.fixture(params=CONFIGS, ids=lambda c: "mt%d_s%d" % c)
def forced_midm(request):
    from gptq_triton_amd import _lib
    lib = _lib.load()
    lib.gptq4_set_midm_tuning(2, *request.param)
    yield lib
    lib.gptq4_set_midm_tuning(1, 0, 0)


@pytest.mark.parametrize("k,n,g", [(2048, 512, 128), (1536, 256, -1), (4096, 256, 512)])
@pytest.mark.parametrize("m", [17, 32, 33, 64, 100, 129, 300])
def test_midm_matmul(forced_midm, k, n, g, m):
    L = O.make_layer(k, n, g, seed=k + n + m, bias=(m % 2 == 0))
    x = O.make_x(m, k, seed=m + 5)
    D = to_dev(L)
    xd = torch.from_numpy(x).cuda()
    y = gptq().matmul4(k if g == -1 else g, xd, D["qweight"], D["scales"], D["qzeros"], D.get("bias"))
    y2 = gptq().matmul4(k if g == -1 else g, xd, D["qweight"], D["scales"], D["qzeros"], D.get("bias"))
    assert torch.equal(y, y2), "the reduction order is fixed: two runs give the same bits"
    ref = O.quant_matmul_ref(x, L["qweight"], L["qzeros"], L["scales"], g, bias=L["bias"])
    if L["bias"] is None:
        assert_close(y.cpu().numpy(), ref, f"mid-M matmul K={k} N={n} g={g} M={m}")
    else:
        ok, max_abs, _ = O.within_tolerance(y.cpu().numpy(), ref)
        assert ok, max_abs


def test_midm_leaves_the_workspace_head_zero(forced_midm):
    from gptq_triton_amd import _lib
    k, n, g = 4096, 512, 128
    L = O.make_layer(k, n, g, seed=1)
    D = to_dev(L)
    xd = torch.from_numpy(O.make_x(40, k, seed=2)).cuda()
    gptq().matmul4(g, xd, D["qweight"], D["scales"], D["qzeros"])
    ws = _lib.workspace(xd.device, 0)
    torch.cuda.synchronize()
    assert int(ws[:_lib.WS_HEAD_BYTES].view(torch.int32).abs().sum()) == 0


def test_midm_one_hot_rows_reproduce_weight_rows(forced_midm):
    """x = e_k picks row k of the dequantised weight: exact, whatever wave and K slice row k falls in."""
    k, n, g = 1024, 256, 128
    L = O.make_layer(k, n, g, seed=9)
    D = to_dev(L)
    rows = np.array([0, 1, 7, 8, 63, 64, 255, 256, 300, 511, 512, 700, 767, 768, 1000, 1023] * 2 + [5, 130])
    x = np.zeros((len(rows), k), dtype=np.float16)
    x[np.arange(len(rows)), rows] = 1.0
    y = gptq().matmul4(g, torch.from_numpy(x).cuda(), D["qweight"], D["scales"], D["qzeros"])
    W = O.dequant_fp16(L["qweight"], L["qzeros"], L["scales"], g)
    assert (y.cpu().numpy().view(np.uint16) == W[rows].view(np.uint16)).all()


@pytest.mark.parametrize("g", [-1, 128])
@pytest.mark.parametrize("m", [17, 64, 150])
def test_midm_gateup(forced_midm, g, m):
    k, n = 1024, 2816
    gate = O.make_layer(k, n, g, seed=100)
    up = O.make_layer(k, n, g, seed=101)
    x = O.make_x(m, k, seed=102 + m)
    Dg, Du = to_dev(gate), to_dev(up)
    h = gptq().llama_mlp_4(k if g == -1 else g, torch.from_numpy(x).cuda(), Dg["qweight"], Dg["scales"], Dg["qzeros"],
                           Du["qweight"], Du["scales"], Du["qzeros"])
    ref = O.mlp_gateup_ref(x, (gate["qweight"], gate["qzeros"], gate["scales"]),
                           (up["qweight"], up["qzeros"], up["scales"]), g)
    assert_close(h.cpu().numpy(), ref, f"mid-M gate/up g={g} M={m}")


@pytest.mark.parametrize("b,s,pos0,g", [(1, 17, 2030, -1), (2, 33, 10, 128), (40, 1, 500, 128), (3, 50, 7, 128)])
def test_midm_qkv_rotary(forced_midm, b, s, pos0, g):
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
        assert_close(got.cpu().numpy(), ref, f"mid-M {name} b={b} s={s} g={g}")


def test_midm_places_cache_rows_by_position(forced_midm):
    from gptq_triton_amd.fused_attention import KV_AT_POSITION
    H, Dh, hidden, g = 8, 128, 1024, 128
    L = O.make_layer(hidden, 3 * hidden, g, seed=320)
    D = to_dev(L)
    G = gptq()
    cos, sin = G.RotaryTable(Dh, 2048).get(torch.device("cuda"), 2048)
    b, s, cap = 3, 11, 64
    rng = np.random.default_rng(321)
    pos = np.stack([rng.permutation(cap)[:s] for _ in range(b)]).astype(np.int64)
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


def test_midm_and_tiled_kernels_agree_within_rounding():
    """Both kernels multiply the same fp16 weights; only the fp32 summation order differs."""
    from gptq_triton_amd import _lib
    lib = _lib.load()
    k, n, g, m = 4096, 1024, 128, 96
    L = O.make_layer(k, n, g, seed=5)
    D = to_dev(L)
    xd = torch.from_numpy(O.make_x(m, k, seed=6)).cuda()
    try:
        lib.gptq4_set_midm_tuning(0, 0, 0)
        y0 = gptq().matmul4(g, xd, D["qweight"], D["scales"], D["qzeros"]).float()
        lib.gptq4_set_midm_tuning(2, 0, 0)
        y1 = gptq().matmul4(g, xd, D["qweight"], D["scales"], D["qzeros"]).float()
    finally:
        lib.gptq4_set_midm_tuning(1, 0, 0)
    big = torch.maximum(y0.abs(), y1.abs()).cpu().numpy().astype(np.float16)
    ulp = torch.from_numpy(np.spacing(big).astype(np.float32)).cuda()
    assert bool(((y0 - y1).abs() <= ulp + 1e-4).all())


def test_act_order_inputs_reach_the_mid_m_kernel_through_the_staged_copy():
    """The mid-M kernel has no act-order gather of its own: the call gathers the rows into the
    workspace first, so a permutation gives the right answer with the mid-M kernel forced too; with a
    workspace that has no room for the copy the call still answers (the tiled kernel's own gather)."""
    from gptq_triton_amd import _lib
    lib = _lib.load()
    k, n, g, m = 2048, 512, 128, 48
    L = O.make_layer(k, n, g, seed=21, act_order=True)
    x = O.make_x(m, k, seed=m + 1)
    G = gptq()
    Wq, perm = G.prepare_act_order(torch.from_numpy(L["qweight"]).cuda(), torch.from_numpy(L["g_idx"]).cuda(), g)
    D = to_dev(L)
    xd = torch.from_numpy(x).cuda()
    y = torch.empty((m, n), dtype=torch.float16, device="cuda")
    ws = _lib.workspace(xd.device, lib.gptq4_workspace_bytes(_lib.OP_MATMUL | _lib.OP_WITH_PERM, m, k, n))
    try:
        lib.gptq4_set_midm_tuning(2, 0, 0)
        rc = lib.gptq4_matmul(xd.data_ptr(), Wq.data_ptr(), D["qzeros"].data_ptr(), D["scales"].data_ptr(), perm.data_ptr(), None,
                              y.data_ptr(), m, k, n, g, ws.data_ptr(), ws.numel(), _lib.current_stream(xd.device))
    finally:
        lib.gptq4_set_midm_tuning(1, 0, 0)
    assert rc == 0
    ref = O.quant_matmul_ref(x, L["qweight"], L["qzeros"], L["scales"], g, g_idx=L["g_idx"])
    assert_close(y.cpu().numpy(), ref, "act-order through the C ABI, M=48")
    need = lib.gptq4_workspace_bytes(_lib.OP_MATMUL | _lib.OP_WITH_PERM, m, k, n)
    assert need >= _lib.WS_HEAD_BYTES + m * k * 2
    # a workspace sized for a call without `perm`: room for any partial sums, none promised for the rows
    y.zero_()
    rc = lib.gptq4_matmul(xd.data_ptr(), Wq.data_ptr(), D["qzeros"].data_ptr(), D["scales"].data_ptr(), perm.data_ptr(), None,
                          y.data_ptr(), m, k, n, g, ws.data_ptr(), lib.gptq4_workspace_bytes(_lib.OP_MATMUL, m, k, n),
                          _lib.current_stream(xd.device))
    assert rc == 0
    assert_close(y.cpu().numpy(), ref, "act-order through the C ABI, M=48, no room for the gathered rows")


def test_tile_counts_just_above_a_whole_number_of_rounds_share_their_last_strips():
    """More tiles than CUs, fewer than one and a half times as many: the last column strips (every row tile of them) are
    shared by two workgroups along K inside the launch.  Against the oracle, against the same plan without the sharing
    (`gptq4_set_gemm_tuning(400, 0)`; another summation order in the shared strips, the same bits elsewhere), and a row
    keeps its bits wherever it sits in the batch."""
    from gptq_triton_amd import _lib
    lib = _lib.load()
    G = gptq()
    g = 128
    # gate/up: 88 strips x 4 row tiles = 352 tiles
    k, n, m = 2048, 5632, 200
    gate, up = O.make_layer(k, n, g, seed=400), O.make_layer(k, n, g, seed=401)
    Dg, Du = to_dev(gate), to_dev(up)
    x = O.make_x(m, k, seed=402)
    xd = torch.from_numpy(x).cuda()
    run = lambda xx: G.llama_mlp_4(g, xx, Dg["qweight"], Dg["scales"], Dg["qzeros"], Du["qweight"], Du["scales"], Du["qzeros"])
    h = run(xd)
    assert torch.equal(h, run(xd))
    perm = torch.randperm(m, generator=torch.Generator().manual_seed(3)).cuda()
    assert torch.equal(run(xd[perm]), h[perm])
    ref = O.mlp_gateup_ref(x, (gate["qweight"], gate["qzeros"], gate["scales"]), (up["qweight"], up["qzeros"], up["scales"]), g)
    assert_close(h.cpu().numpy(), ref, "gate/up, shared last strips")
    try:
        lib.gptq4_set_gemm_tuning(400, 0)
        h0 = run(xd)
    finally:
        lib.gptq4_set_gemm_tuning(0, 0)
    assert_close(h0.cpu().numpy(), ref, "gate/up, no sharing")
    whole = (352 - 96) // 4 * 64          # columns of the strips that stay whole: 256 CUs -> 96 tiles = 24 strips shared
    assert torch.equal(h[:, :whole], h0[:, :whole]) and not torch.equal(h[:, whole:], h0[:, whole:])

    # QKV + rotary: 48 heads' strips x 7 row tiles = 336 tiles
    hidden, heads, m = 2048, 16, 400
    L = O.make_layer(hidden, 3 * hidden, g, seed=410)
    D = to_dev(L)
    x = O.make_x(m, hidden, seed=411).reshape(1, m, hidden)
    pos = np.arange(m)[None, :].astype(np.int32)
    cos, sin = G.RotaryTable(128, 512).get(torch.device("cuda"), 512)
    q, kk, v = G.qkv_rotary(g, torch.from_numpy(x).cuda(), D["qweight"], D["scales"], D["qzeros"], torch.from_numpy(pos).cuda(), cos, sin, heads)
    qr, kr, vr = O.qkv_rotary_ref(x, L["qweight"], L["qzeros"], L["scales"], g, pos, heads, 128, max_pos=512)
    for got, want, name in ((q, qr, "q"), (kk, kr, "k"), (v, vr, "v")):
        assert_close(got.cpu().numpy(), want, f"{name}, shared last strips")

    # a plain projection with four waves per workgroup: 96 strips x 3 row tiles = 288 tiles
    k, n, m = 2048, 6144, 150
    L = O.make_layer(k, n, g, seed=420, bias=True)
    D = to_dev(L)
    x = O.make_x(m, k, seed=421)
    try:
        lib.gptq4_set_midm_tuning(2, 100, 0)
        y = G.matmul4(g, torch.from_numpy(x).cuda(), D["qweight"], D["scales"], D["qzeros"], D["bias"])
    finally:
        lib.gptq4_set_midm_tuning(1, 0, 0)
    ok, max_abs, _ = O.within_tolerance(y.cpu().numpy(), O.quant_matmul_ref(x, L["qweight"], L["qzeros"], L["scales"], g, bias=L["bias"]))
    assert ok, max_abs
    from gptq_triton_amd import _lib as L_
    ws = L_.workspace(torch.device("cuda", torch.cuda.current_device()), 0)
    torch.cuda.synchronize()
    assert int(ws[:L_.WS_HEAD_BYTES].view(torch.int32).abs().sum()) == 0
