"""GPU tests of the chained decode launch (gptq4_decode_chain): every phase kind against the oracle, the
o_proj -> add + RMSNorm -> gate/up + SiLU*mul -> down_proj chain stage by stage, determinism from launch to
launch, HIP-graph replays, and the bounded waits giving up cleanly when a workgroup never reports."""
import numpy as np
import pytest
import torch

from conftest import to_dev
from oracle import gptq_oracle as O
from test_gpu_parity import assert_close

pytestmark = pytest.mark.gpu


def _chain():
    from gptq_triton_amd import chain
    return chain


def _trip(L):
    return L["qweight"], L["qzeros"], L["scales"]


@pytest.fixture(autouse=True)
def short_waits():
    """A launch that cannot complete gives up after about a second instead of the default several."""
    from gptq_triton_amd import _lib
    lib = _lib.load()
    lib.gptq4_set_chain_tuning(0, 0, 1 << 19, -1)
    yield lib
    lib.gptq4_set_chain_tuning(0, 0, 0, -1)


@pytest.mark.parametrize("m", [1, 3, 4])
@pytest.mark.parametrize("k,n,g", [(256, 256, 128), (1024, 2816, 128), (4096, 4096, -1), (11008, 4096, 128)])
def test_single_projection_phase(m, k, n, g):
    C = _chain()
    L = O.make_layer(k, n, g, seed=k + n, bias=(k == 1024))
    D = to_dev(L)
    x = O.make_x(m, k, seed=m)
    xd = torch.from_numpy(x).cuda()
    y = torch.full((m, n), float("nan"), dtype=torch.float16, device="cuda")
    ph = C.projection(D["qweight"], D["qzeros"], D["scales"], g, x=xd, output=C.OUT_ROWS, y=y, bias=D.get("bias"))
    ws = C.decode_chain([ph], m, xd.device)
    torch.cuda.synchronize()
    assert C.error_word(ws) == 0
    ref = O.quant_matmul_ref(x, *_trip(L), g, bias=L["bias"])
    if L["bias"] is None:
        assert_close(y.cpu().numpy(), ref, f"chain projection M={m} K={k} N={n}")
    else:
        # the reference's rounding structure: fp16(sums), then an fp16 add of the bias (quant_linear.py:225,280-281):
        # one ulp of the value before the bias plus one of the result
        ok, max_abs, _ = O.within_tolerance(y.cpu().numpy(), ref)
        assert ok, max_abs
        w16 = O.dequant_fp16(*_trip(L), g)
        ref16, pre16 = O.matmul_fp16(x, w16, L["bias"]), O.matmul_fp16(x, w16)
        diff = np.abs(y.cpu().numpy().astype(np.float32) - ref16.astype(np.float32))
        assert (diff <= np.spacing(np.abs(ref16)).astype(np.float32) + np.spacing(np.abs(pre16)).astype(np.float32)).all()


@pytest.mark.parametrize("m", [1, 4])
@pytest.mark.parametrize("k,n,g", [(512, 768, 128), (4096, 11008, 128)])
def test_gate_up_pair_phase(m, k, n, g):
    C = _chain()
    gate, up = O.make_layer(k, n, g, seed=1), O.make_layer(k, n, g, seed=2)
    Dg, Du = to_dev(gate), to_dev(up)
    x = O.make_x(m, k, seed=10 + m)
    xd = torch.from_numpy(x).cuda()
    h = torch.full((m, n), float("nan"), dtype=torch.float16, device="cuda")
    ph = C.projection(Dg["qweight"], Dg["qzeros"], Dg["scales"], g, up=(Du["qweight"], Du["qzeros"], Du["scales"]),
                      x=xd, output=C.OUT_ROWS, y=h)
    C.decode_chain([ph], m, xd.device)
    ref = O.mlp_gateup_ref(x, _trip(gate), _trip(up), g)
    assert_close(h.cpu().numpy(), ref, f"chain gate/up M={m} K={k} I={n}")


@pytest.mark.parametrize("m", [1, 2, 4])
@pytest.mark.parametrize("hidden,heads,g,at_position", [(1024, 8, 128, False), (4096, 32, -1, True)])
def test_qkv_rotary_phase(m, hidden, heads, g, at_position):
    import gptq_triton_amd as G
    C = _chain()
    L = O.make_layer(hidden, 3 * hidden, g, seed=77)
    D = to_dev(L)
    x = O.make_x(m, hidden, seed=20 + m)
    xd = torch.from_numpy(x).cuda()
    pos = (np.arange(m) * 7 + 2040 - 7 * m).astype(np.int32)
    cos, sin = G.RotaryTable(128, 2048).get(torch.device("cuda"), 2048)
    cap = 2048 if at_position else 1
    q = torch.zeros((m, heads, 1, 128), dtype=torch.float16, device="cuda")
    kc = torch.full((m, heads, cap, 128), 7.0, dtype=torch.float16, device="cuda")
    vc = torch.full((m, heads, cap, 128), 7.0, dtype=torch.float16, device="cuda")
    rope = dict(position_ids=torch.from_numpy(pos).cuda(), cos=cos, sin=sin, q=q, k=kc, v=vc, heads=heads,
                kv_offset=-1 if at_position else 0)
    ph = C.projection(D["qweight"], D["qzeros"], D["scales"], g, x=xd, output=C.OUT_ROPE, rope=rope)
    C.decode_chain([ph], m, xd.device)
    qr, kr, vr = O.qkv_rotary_ref(x.reshape(m, 1, hidden), *_trip(L), g, pos.reshape(m, 1), heads, 128, max_pos=2048)
    assert_close(q.cpu().numpy(), qr, "chain qkv: q")
    if at_position:
        rows = torch.from_numpy(pos.astype(np.int64)).cuda()
        k_new = torch.stack([kc[b, :, rows[b]] for b in range(m)])[:, :, None]
        v_new = torch.stack([vc[b, :, rows[b]] for b in range(m)])[:, :, None]
        # only the token's row of the cache was written
        assert int((kc != 7.0).any(-1).sum()) <= m * heads and int((vc != 7.0).any(-1).sum()) <= m * heads
    else:
        k_new, v_new = kc, vc
    assert_close(k_new.cpu().numpy(), kr, "chain qkv: k")
    assert_close(v_new.cpu().numpy(), vr, "chain qkv: v")
    # and the bits of the stand-alone entry point's rotary arithmetic on the same sums are not required; its values are
    q0, k0, v0 = G.qkv_rotary(L["qweight"].shape[0] * 8 if g == -1 else g, xd.view(m, 1, hidden), D["qweight"], D["scales"], D["qzeros"],
                              torch.from_numpy(pos).cuda().view(m, 1), cos, sin, heads)
    assert (q.float() - q0.float()).abs().max().item() <= 2e-2


def mlp_chain(C, D, xd, hd, wd, eps, m, hidden, inter, g, outputs=True):
    """o_proj(x) -> h + o, RMSNorm -> gate/up -> down; returns the tensors the launch writes."""
    out = dict(o=torch.full((m, hidden), float("nan"), dtype=torch.float16, device="cuda") if outputs else None,
               s=torch.full((m, hidden), float("nan"), dtype=torch.float16, device="cuda"),
               act=torch.full((m, inter), float("nan"), dtype=torch.float16, device="cuda") if outputs else None,
               y=torch.full((m, hidden), float("nan"), dtype=torch.float16, device="cuda"))
    o, gate, up, down = D
    phases = [
        C.projection(o["qweight"], o["qzeros"], o["scales"], g, x=xd, output=C.OUT_ROWS if outputs else C.OUT_NONE, y=out["o"]),
        C.projection(gate["qweight"], gate["qzeros"], gate["scales"], g, up=(up["qweight"], up["qzeros"], up["scales"]),
                     input=C.IN_NORM_PREV, x=hd, norm_weight=wd, eps=eps, sum_out=out["s"],
                     output=C.OUT_ROWS if outputs else C.OUT_NONE, y=out["act"]),
        C.projection(down["qweight"], down["qzeros"], down["scales"], g, input=C.IN_PREV, output=C.OUT_ROWS, y=out["y"]),
    ]
    out["ws"] = C.decode_chain(phases, m, xd.device)
    return out


@pytest.mark.parametrize("m", [1, 2, 4])
@pytest.mark.parametrize("hidden,inter,g", [(1024, 2816, 128), (4096, 11008, 128), (5120, 13824, 128), (6656, 17920, 512)])
def test_mlp_chain_stage_by_stage(m, hidden, inter, g):
    from gptq_triton_amd.decoder_ops import rms_norm
    C = _chain()
    layers = [O.make_layer(hidden, hidden, g, seed=31), O.make_layer(hidden, inter, g, seed=32),
              O.make_layer(hidden, inter, g, seed=33), O.make_layer(inter, hidden, g, seed=34)]
    # scales that keep the activations O(1) through the chain
    for L, k in zip(layers, (hidden, hidden, hidden, inter)):
        L["scales"] = (L["scales"].astype(np.float32) * (6.0 / np.sqrt(k))).astype(np.float16)
    D = [to_dev(L) for L in layers]
    rng = np.random.default_rng(m)
    x = O.make_x(m, hidden, seed=40 + m)
    h = (rng.standard_normal((m, hidden)) * 2).astype(np.float16)
    w = (1.0 + 0.1 * rng.standard_normal(hidden)).astype(np.float16)
    xd, hd, wd = (torch.from_numpy(t).cuda() for t in (x, h, w))
    eps = 1e-6
    out = mlp_chain(C, D, xd, hd, wd, eps, m, hidden, inter, g)
    torch.cuda.synchronize()
    assert C.error_word(out["ws"]) == 0
    # stage 1: o_proj
    assert_close(out["o"].cpu().numpy(), O.quant_matmul_ref(x, *_trip(layers[0]), g), "chain: o_proj")
    # stage 2: the residual add is one fp16 add of the fp16 projection
    assert torch.equal(out["s"], hd + out["o"])
    # stage 3: RMSNorm as the stand-alone kernel computes it on the same sums (same thread order, same bits), then gate/up
    xn = rms_norm(out["s"], wd, eps)
    assert_close(out["act"].cpu().numpy(), O.mlp_gateup_ref(xn.cpu().numpy(), _trip(layers[1]), _trip(layers[2]), g), "chain: gate/up")
    # stage 4: down_proj of the chain's own intermediate
    assert_close(out["y"].cpu().numpy(), O.quant_matmul_ref(out["act"].cpu().numpy(), *_trip(layers[3]), g), "chain: down_proj")
    # the same chain without the intermediate outputs, twice: the same bits every time
    for _ in range(2):
        lean = mlp_chain(C, D, xd, hd, wd, eps, m, hidden, inter, g, outputs=False)
        assert torch.equal(lean["y"], out["y"]) and torch.equal(lean["s"], out["s"])


@pytest.mark.parametrize("m", [1, 3])
@pytest.mark.parametrize("hidden,inter,heads,g", [(1024, 2816, 8, 128), (4096, 11008, 32, 128)])
def test_layer_chain_into_the_next_qkv(m, hidden, inter, heads, g):
    """The decoder's order: o_proj -> add + norm -> gate/up -> down -> add + norm -> the NEXT layer's QKV + rotary.
    The second residual add reads the sums of the first, which every workgroup kept in LDS."""
    import gptq_triton_amd as G
    from gptq_triton_amd.decoder_ops import rms_norm
    C = _chain()
    layers = [O.make_layer(hidden, hidden, g, seed=81), O.make_layer(hidden, inter, g, seed=82),
              O.make_layer(hidden, inter, g, seed=83), O.make_layer(inter, hidden, g, seed=84), O.make_layer(hidden, 3 * hidden, g, seed=85)]
    for L, k in zip(layers, (hidden, hidden, hidden, inter, hidden)):
        L["scales"] = (L["scales"].astype(np.float32) * (6.0 / np.sqrt(k))).astype(np.float16)
    o, gate, up, down, qkv = [to_dev(L) for L in layers]
    rng = np.random.default_rng(m)
    x = O.make_x(m, hidden, seed=50 + m)
    h = (rng.standard_normal((m, hidden)) * 2).astype(np.float16)
    w1 = (1.0 + 0.1 * rng.standard_normal(hidden)).astype(np.float16)
    w2 = (1.0 + 0.1 * rng.standard_normal(hidden)).astype(np.float16)
    xd, hd, w1d, w2d = (torch.from_numpy(t).cuda() for t in (x, h, w1, w2))
    pos = torch.arange(m, dtype=torch.int32, device="cuda") * 3 + 11
    cos, sin = G.RotaryTable(128, 2048).get(torch.device("cuda"), 2048)
    new = lambda *shape: torch.full(shape, float("nan"), dtype=torch.float16, device="cuda")
    s1, s2, yd = new(m, hidden), new(m, hidden), new(m, hidden)
    q, k, v = new(m, heads, 1, 128), new(m, heads, 1, 128), new(m, heads, 1, 128)
    phases = [
        C.projection(o["qweight"], o["qzeros"], o["scales"], g, x=xd),
        C.projection(gate["qweight"], gate["qzeros"], gate["scales"], g, up=(up["qweight"], up["qzeros"], up["scales"]),
                     input=C.IN_NORM_PREV, x=hd, norm_weight=w1d, eps=1e-6, sum_out=s1),
        C.projection(down["qweight"], down["qzeros"], down["scales"], g, input=C.IN_PREV, output=C.OUT_ROWS, y=yd),
        C.projection(qkv["qweight"], qkv["qzeros"], qkv["scales"], g, input=C.IN_NORM_PREV, x=s1, norm_weight=w2d, eps=1e-6, sum_out=s2,
                     output=C.OUT_ROPE, rope=dict(position_ids=pos, cos=cos, sin=sin, q=q, k=k, v=v, heads=heads)),
    ]
    ws = C.decode_chain(phases, m, xd.device)
    torch.cuda.synchronize()
    assert C.error_word(ws) == 0
    assert torch.equal(s2, s1 + yd), "the second residual add takes the first one's sums"
    xn = rms_norm(s2, w2d, 1e-6)
    qr, kr, vr = O.qkv_rotary_ref(xn.cpu().numpy().reshape(m, 1, hidden), *_trip(layers[4]), g, pos.cpu().numpy().reshape(m, 1), heads, 128, max_pos=2048)
    assert_close(q.cpu().numpy(), qr, "layer chain: next q")
    assert_close(k.cpu().numpy(), kr, "layer chain: next k")
    assert_close(v.cpu().numpy(), vr, "layer chain: next v")
    # sums of an earlier norm phase than the latest one are not at hand inside the launch
    from gptq_triton_amd import _lib
    bad = list(phases)
    bad[3] = C.projection(qkv["qweight"], qkv["qzeros"], qkv["scales"], g, input=C.IN_NORM_PREV, x=s1, norm_weight=w2d, eps=1e-6,
                          sum_out=s2, output=C.OUT_ROPE, rope=dict(position_ids=pos, cos=cos, sin=sin, q=q, k=k, v=v, heads=heads))
    bad.insert(3, C.projection(o["qweight"], o["qzeros"], o["scales"], g, input=C.IN_NORM_PREV, x=hd, norm_weight=w1d, eps=1e-6,
                               sum_out=new(m, hidden)))
    arr = (_lib.Phase * len(bad))(*bad)
    assert _lib.load().gptq4_chain_workspace_bytes(arr, len(bad), m) == 0


def test_norm_rows_then_qkv_and_many_launches():
    """A first phase that normalises rows from memory (residual + delta), and 50 launches in a row on one workspace:
    the state the launches keep in it carries from one to the next."""
    import gptq_triton_amd as G
    from gptq_triton_amd.decoder_ops import add_rms_norm
    C = _chain()
    m, hidden, heads, g = 2, 1024, 8, 128
    L = O.make_layer(hidden, 3 * hidden, g, seed=5)
    D = to_dev(L)
    rng = np.random.default_rng(0)
    h = (rng.standard_normal((m, hidden)) * 2).astype(np.float16)
    d = rng.standard_normal((m, hidden)).astype(np.float16)
    w = (1.0 + 0.1 * rng.standard_normal(hidden)).astype(np.float16)
    hd, dd, wd = (torch.from_numpy(t).cuda() for t in (h, d, w))
    pos = torch.tensor([5, 9], dtype=torch.int32, device="cuda")
    cos, sin = G.RotaryTable(128, 2048).get(torch.device("cuda"), 2048)
    s_ref, x_ref = add_rms_norm(hd, dd, wd, 1e-6)
    qr, kr, vr = O.qkv_rotary_ref(x_ref.cpu().numpy().reshape(m, 1, hidden), *_trip(L), g, pos.cpu().numpy().reshape(m, 1), heads, 128, max_pos=2048)
    first = None
    for it in range(50):
        q = torch.zeros((m, heads, 1, 128), dtype=torch.float16, device="cuda")
        k = torch.zeros_like(q)
        v = torch.zeros_like(q)
        s = torch.zeros((m, hidden), dtype=torch.float16, device="cuda")
        ph = C.projection(D["qweight"], D["qzeros"], D["scales"], g, input=C.IN_NORM_ROWS, x=hd, delta=dd, norm_weight=wd, eps=1e-6,
                          sum_out=s, output=C.OUT_ROPE, rope=dict(position_ids=pos, cos=cos, sin=sin, q=q, k=k, v=v, heads=heads))
        ws = C.decode_chain([ph], m, hd.device)
        if first is None:
            first = (q, k, v)
            assert torch.equal(s, s_ref)
            assert_close(q.cpu().numpy(), qr, "chain norm + qkv: q")
            assert_close(v.cpu().numpy(), vr, "chain norm + qkv: v")
        else:
            assert torch.equal(q, first[0]) and torch.equal(k, first[1]) and torch.equal(v, first[2])
    assert C.error_word(ws) == 0
    assert int(ws[:4].view(torch.int32).item()) >= 50, "the state counts the launches"


def test_chain_replays_in_a_graph():
    C = _chain()
    m, hidden, inter, g = 1, 1024, 2816, 128
    layers = [O.make_layer(hidden, hidden, g, seed=61), O.make_layer(hidden, inter, g, seed=62),
              O.make_layer(hidden, inter, g, seed=63), O.make_layer(inter, hidden, g, seed=64)]
    D = [to_dev(L) for L in layers]
    xd = torch.from_numpy(O.make_x(m, hidden, seed=1)).cuda()
    hd = torch.from_numpy(O.make_x(m, hidden, seed=2)).cuda()
    wd = torch.ones(hidden, dtype=torch.float16, device="cuda")
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        eager = mlp_chain(C, D, xd, hd, wd, 1e-6, m, hidden, inter, g, outputs=False)
        want = eager["y"].clone()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            cap = mlp_chain(C, D, xd, hd, wd, 1e-6, m, hidden, inter, g, outputs=False)
    torch.cuda.current_stream().wait_stream(side)
    for i in range(5):
        cap["y"].zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(cap["y"], want), f"replay {i}"
        # eager launches between the replays share the stream's workspace state
        again = mlp_chain(C, D, xd, hd, wd, 1e-6, m, hidden, inter, g, outputs=False)
        assert torch.equal(again["y"], want)


def test_bounded_wait_gives_up_and_the_error_is_sticky(short_waits):
    """Workgroup 0 never stores its partial sums (a host-side test hook): every poll for them runs into its limit, every
    workgroup returns, the launch ends normally with the error word set; later launches on that workspace return
    at once until the workspace is cleared."""
    C = _chain()
    lib = short_waits
    m, hidden, inter, g = 1, 512, 768, 128
    layers = [O.make_layer(hidden, hidden, g, seed=71), O.make_layer(hidden, inter, g, seed=72),
              O.make_layer(hidden, inter, g, seed=73), O.make_layer(inter, hidden, g, seed=74)]
    D = [to_dev(L) for L in layers]
    xd = torch.from_numpy(O.make_x(m, hidden, seed=1)).cuda()
    hd = torch.from_numpy(O.make_x(m, hidden, seed=2)).cuda()
    wd = torch.ones(hidden, dtype=torch.float16, device="cuda")
    good = mlp_chain(C, D, xd, hd, wd, 1e-6, m, hidden, inter, g, outputs=False)
    torch.cuda.synchronize()
    ws = good["ws"]
    assert C.error_word(ws) == 0
    lib.gptq4_set_chain_tuning(0, 0, 64, 0)           # 64 polls, workgroup 0 silent
    try:
        mlp_chain(C, D, xd, hd, wd, 1e-6, m, hidden, inter, g, outputs=False)
        torch.cuda.synchronize()                        # returns: nobody waits for ever
    finally:
        lib.gptq4_set_chain_tuning(0, 0, 1 << 19, -1)
    assert C.error_word(ws) == 1
    after = mlp_chain(C, D, xd, hd, wd, 1e-6, m, hidden, inter, g, outputs=False)
    torch.cuda.synchronize()
    assert C.error_word(ws) == 1 and bool(torch.isnan(after["y"].float()).all()), "a launch on a failed workspace must do nothing"
    ws.zero_()
    fresh = mlp_chain(C, D, xd, hd, wd, 1e-6, m, hidden, inter, g, outputs=False)
    torch.cuda.synchronize()
    assert C.error_word(ws) == 0 and torch.equal(fresh["y"], good["y"])


def test_chain_argument_errors():
    from gptq_triton_amd import _lib
    C = _chain()
    lib = _lib.load()
    L = to_dev(O.make_layer(256, 256, 128, seed=1))
    x = torch.zeros((1, 256), dtype=torch.float16, device="cuda")
    y = torch.zeros((1, 256), dtype=torch.float16, device="cuda")
    ok = C.projection(L["qweight"], L["qzeros"], L["scales"], 128, x=x, output=C.OUT_ROWS, y=y)
    arr = (_lib.Phase * 1)(ok)
    assert lib.gptq4_chain_workspace_bytes(arr, 1, 1) > 8192
    assert lib.gptq4_chain_workspace_bytes(arr, 1, 5) == 0                      # too many rows
    assert lib.gptq4_decode_chain(arr, 1, 5, None, 0, None) == -2
    assert lib.gptq4_decode_chain(arr, 1, 1, None, 0, None) == -4              # no workspace
    nobody_reads = C.projection(L["qweight"], L["qzeros"], L["scales"], 128, x=x)
    arr = (_lib.Phase * 1)(nobody_reads)
    assert lib.gptq4_decode_chain(arr, 1, 1, None, 0, None) == -2
    first_from_prev = C.projection(L["qweight"], L["qzeros"], L["scales"], 128, input=C.IN_PREV, output=C.OUT_ROWS, y=y)
    arr = (_lib.Phase * 1)(first_from_prev)
    assert lib.gptq4_decode_chain(arr, 1, 1, None, 0, None) == -2
