"""GPU parity at the full sizes of the five benchmark workloads (LLaMA-7B q_proj, fused 7B MLP,
fused 7B QKV + rotary, 13B layer shapes with act-order, 30B layer shapes with groupsize 512).

The HIP path always computes every row.  Where the CPU oracle would need minutes for all of
them, it is evaluated on a seeded sample of rows (rows of a matmul are independent), and the
rest is covered by two size-independent properties of the operator:

* permuting the rows of x permutes the rows of the result bit for bit (any row-indexing or
  tile-placement error shows up, wherever it is);
* one-hot rows return rows of the dequantised weight matrix exactly.
"""
import functools

import numpy as np
import pytest
import torch

from conftest import bits, to_dev
from oracle import gptq_oracle as O
from test_gpu_parity import assert_close, gptq

pytestmark = pytest.mark.gpu


def sample_rows(m, count, seed):
    """First, last and tile-boundary rows plus a seeded random sample."""
    if m <= count:
        return np.arange(m)
    fixed = [r for r in (0, 1, 15, 16, 17, 31, 32, 63, 64, 127, 128, 129, 255, 256, 767, 768, m - 2, m - 1) if r < m]
    rng = np.random.default_rng(seed)
    extra = rng.choice(m, size=count, replace=False)
    return np.unique(np.concatenate([np.array(fixed, dtype=np.int64), extra]))


@functools.lru_cache(maxsize=3)
def layer_and_weights(k, n, g, seed, act_order=False):
    """Seeded layer and its oracle-dequantised fp16 weights (kept for the next M of the same shape)."""
    L = O.make_layer(k, n, g, seed=seed, act_order=act_order)
    return L, O.dequant_fp16(L["qweight"], L["qzeros"], L["scales"], g, L["g_idx"])


def quant_linear(L, k, n, g, act_order=False):
    G = gptq()
    q = G.QuantLinear(4, g, k, n, bias=False, act_order=act_order)
    q.qweight, q.qzeros, q.scales = (torch.from_numpy(L[t]) for t in ("qweight", "qzeros", "scales"))
    if act_order:
        q.g_idx = torch.from_numpy(L["g_idx"])
    return q


# ------------------------------------------------- workload 0: single QuantLinear, q_proj shape
@pytest.mark.parametrize("m", [1, 128])
def test_q_proj_7b(m):
    k = n = 4096
    L = O.make_layer(k, n, -1, seed=1000)
    x = O.make_x(m, k, seed=1001 + m)
    assert L["qweight"].shape == (512, 4096) and L["qzeros"].shape == (1, 512) and L["scales"].shape == (1, 4096)
    D = to_dev(L)
    y = gptq().matmul4(k, torch.from_numpy(x).cuda(), D["qweight"], D["scales"], D["qzeros"])
    assert_close(y.cpu().numpy(), O.quant_matmul_ref(x, L["qweight"], L["qzeros"], L["scales"], -1), f"q_proj M={m}")


# ------------------------------------------------------------- workload 1: fused 7B MLP, g=128
@pytest.fixture(scope="module")
def mlp_7b():
    k, n, g = 4096, 11008, 128
    raw = {}
    layers = {}
    for name, (ki, ni), seed in (("gate_proj", (k, n), 1100), ("up_proj", (k, n), 1101), ("down_proj", (n, k), 1102)):
        L = O.make_layer(ki, ni, g, seed=seed)
        raw[name] = (L["qweight"], L["qzeros"], L["scales"])
        layers[name] = quant_linear(L, ki, ni, g)
    mlp = gptq().QuantLlamaMLP(layers["gate_proj"], layers["down_proj"], layers["up_proj"]).cuda()
    return mlp, raw


@pytest.mark.parametrize("m", [1, 16, 512])
def test_mlp_7b(mlp_7b, m):
    mlp, raw = mlp_7b
    g = 128
    x = O.make_x(m, 4096, seed=1110 + m)
    xd = torch.from_numpy(x).cuda()
    h = mlp.gate_up(xd)
    y = mlp(xd)
    rows = sample_rows(m, 40, seed=m)
    h_ref = O.mlp_gateup_ref(x[rows], raw["gate_proj"], raw["up_proj"], g)
    assert_close(h[rows].cpu().numpy(), h_ref, f"7B MLP gate/up M={m}")
    # the down projection is judged on the kernel's own fp16 intermediate, so a one-ulp
    # difference in h is not counted twice
    y_ref = O.quant_matmul_ref(h[rows].cpu().numpy(), *raw["down_proj"], g)
    assert_close(y[rows].cpu().numpy(), y_ref, f"7B MLP down M={m}")
    if m > 16:
        p = torch.from_numpy(np.random.default_rng(5).permutation(m)).cuda()
        assert torch.equal(mlp.gate_up(xd[p]), h[p]) and torch.equal(mlp(xd[p]), y[p])


# ------------------------------------------------------ workload 2: fused 7B QKV + rotary, g=-1
@pytest.fixture(scope="module")
def qkv_7b():
    hidden = 4096
    L = O.make_layer(hidden, 3 * hidden, -1, seed=1200)
    return L, to_dev(L)


def test_qkv_rotary_7b_decode_at_position_2047(qkv_7b):
    L, D = qkv_7b
    hidden, H, Dh = 4096, 32, 128
    G = gptq()
    cos, sin = G.RotaryTable(Dh, 2048).get(torch.device("cuda"), 2048)
    x = O.make_x(1, hidden, seed=1201).reshape(1, 1, hidden)
    pos = np.array([[2047]], dtype=np.int64)
    q, k, v = G.qkv_rotary(hidden, torch.from_numpy(x).cuda(), D["qweight"], D["scales"], D["qzeros"],
                           torch.from_numpy(pos).cuda(), cos, sin, H, Dh)
    qr, kr, vr = O.qkv_rotary_ref(x, L["qweight"], L["qzeros"], L["scales"], -1, pos, H, Dh, max_pos=2048)
    for got, ref, name in ((q, qr, "q"), (k, kr, "k"), (v, vr, "v")):
        assert got.shape == (1, H, 1, Dh)
        assert_close(got.cpu().numpy(), ref, f"7B qkv decode {name}")


def test_qkv_rotary_7b_prefill_2048(qkv_7b):
    L, D = qkv_7b
    hidden, H, Dh, S = 4096, 32, 128, 2048
    G = gptq()
    cos, sin = G.RotaryTable(Dh, 2048).get(torch.device("cuda"), 2048)
    x = O.make_x(S, hidden, seed=1202).reshape(1, S, hidden)
    pos = np.arange(S, dtype=np.int64)[None, :]
    xd, pd = torch.from_numpy(x).cuda(), torch.from_numpy(pos).cuda()
    q, k, v = G.qkv_rotary(hidden, xd, D["qweight"], D["scales"], D["qzeros"], pd, cos, sin, H, Dh)
    rows = sample_rows(S, 40, seed=7)
    qr, kr, vr = O.qkv_rotary_ref(x[:, rows], L["qweight"], L["qzeros"], L["scales"], -1, pos[:, rows], H, Dh,
                                  max_pos=2048)
    for got, ref, name in ((q, qr, "q"), (k, kr, "k"), (v, vr, "v")):
        assert got.shape == (1, H, S, Dh)
        assert_close(got[:, :, rows].cpu().numpy(), ref, f"7B qkv prefill {name}")
    # tokens (with their positions) in another order give the same rows, bit for bit
    p = torch.from_numpy(np.random.default_rng(8).permutation(S)).cuda()
    q2, k2, v2 = G.qkv_rotary(hidden, xd[:, p].contiguous(), D["qweight"], D["scales"], D["qzeros"],
                              pd[:, p].contiguous(), cos, sin, H, Dh)
    assert torch.equal(q2, q[:, :, p]) and torch.equal(k2, k[:, :, p]) and torch.equal(v2, v[:, :, p])


# ----------------------------------------- workload 3: 13B layer shapes, g=128, act-order
@pytest.mark.parametrize("k,n", [(5120, 5120), (13824, 5120)])
@pytest.mark.parametrize("m", [1, 2048])
def test_13b_act_order_linear(k, n, m):
    g = 128
    L, W = layer_and_weights(k, n, g, 1300 + k // 128, True)
    layer = quant_linear(L, k, n, g, act_order=True).cuda()
    x = O.make_x(m, k, seed=1301 + m)
    xd = torch.from_numpy(x).cuda()
    y = layer(xd)
    rows = sample_rows(m, 24, seed=k)
    assert_close(y[rows].cpu().numpy(), O.matmul_ref(x[rows], W), f"13B act-order K={k} N={n} M={m}")
    if m > 16:
        p = torch.from_numpy(np.random.default_rng(9).permutation(m)).cuda()
        assert torch.equal(layer(xd[p]), y[p])


@pytest.mark.parametrize("m", [1, 2048])
def test_13b_act_order_mlp_gateup(m):
    k, n, g = 5120, 13824, 128
    gate = O.make_layer(k, n, g, seed=1310, act_order=True)
    up = O.make_layer(k, n, g, seed=1311)
    up["g_idx"] = gate["g_idx"]                    # gate and up read one input, hence one g_idx
    down = O.make_layer(n, k, g, seed=1312, act_order=True)
    mlp = gptq().QuantLlamaMLP(quant_linear(gate, k, n, g, True), quant_linear(down, n, k, g, True),
                               quant_linear(up, k, n, g, True)).cuda()
    x = O.make_x(m, k, seed=1313 + m)
    h = mlp.gate_up(torch.from_numpy(x).cuda())
    rows = sample_rows(m, 16, seed=m + 1)
    ref = O.mlp_gateup_ref(x[rows], (gate["qweight"], gate["qzeros"], gate["scales"], gate["g_idx"]),
                           (up["qweight"], up["qzeros"], up["scales"], up["g_idx"]), g)
    assert_close(h[rows].cpu().numpy(), ref, f"13B act-order gate/up M={m}")


@pytest.mark.parametrize("gate_act_order", [True, False])
@pytest.mark.parametrize("m", [1, 8, 48, 300])
def test_act_order_mlp_forward_chains_into_down_proj_without_a_gather(m, gate_act_order):
    """forward() lays the gate/up output columns out in the order of down_proj's sorted rows: the result must be
    the very bits of down_proj(gate_up(x)), which gathers the intermediate, and meet the oracle's bar."""
    k, n, g = 1024, 2560, 128
    gate = O.make_layer(k, n, g, seed=1330, act_order=gate_act_order)
    up = O.make_layer(k, n, g, seed=1331)
    up["g_idx"] = gate["g_idx"]
    down = O.make_layer(n, k, g, seed=1332, act_order=True)
    mlp = gptq().QuantLlamaMLP(quant_linear(gate, k, n, g, gate_act_order), quant_linear(down, n, k, g, True),
                               quant_linear(up, k, n, g, gate_act_order)).cuda()
    x = O.make_x(m, k, seed=1333 + m)
    xd = torch.from_numpy(x).cuda()
    mid = mlp.gate_up(xd)
    two_step = mlp.down_proj(mid)
    y = mlp(xd)
    assert torch.equal(y, two_step)
    ref = O.quant_matmul_ref(mid.cpu().numpy(), down["qweight"], down["qzeros"], down["scales"], g, g_idx=down["g_idx"])
    assert_close(y.cpu().numpy(), ref, f"act-order MLP forward M={m}")
    if m <= 4:
        w = torch.from_numpy(np.random.default_rng(5).standard_normal(k).astype(np.float16)).cuda()
        delta = torch.from_numpy(O.make_x(m, k, seed=77)).cuda()
        s, y2 = mlp.forward_normed(xd, delta, w, 1e-6)
        s_ref, normed = gptq().add_rms_norm(xd, delta, w, 1e-6)
        assert torch.equal(s, s_ref) and torch.equal(y2, mlp(normed))


def test_13b_act_order_qkv_rotary():
    hidden, H, Dh, g, S = 5120, 40, 128, 128, 2048
    L = O.make_layer(hidden, 3 * hidden, g, seed=1320, act_order=True)
    G = gptq()
    D = to_dev(L)
    qs, perm = G.prepare_act_order(D["qweight"], D["g_idx"], g)
    cos, sin = G.RotaryTable(Dh, 2048).get(torch.device("cuda"), 2048)
    for s, pos0 in ((1, 2047), (S, 0)):
        x = O.make_x(s, hidden, seed=1321 + s).reshape(1, s, hidden)
        pos = (pos0 + np.arange(s, dtype=np.int64))[None, :]
        q, k, v = G.qkv_rotary(g, torch.from_numpy(x).cuda(), qs, D["scales"], D["qzeros"],
                               torch.from_numpy(pos).cuda(), cos, sin, H, Dh, perm=perm)
        rows = sample_rows(s, 16, seed=s)
        qr, kr, vr = O.qkv_rotary_ref(x[:, rows], L["qweight"], L["qzeros"], L["scales"], g, pos[:, rows], H, Dh,
                                      g_idx=L["g_idx"], max_pos=2048)
        for got, ref, name in ((q, qr, "q"), (k, kr, "k"), (v, vr, "v")):
            assert_close(got[:, :, rows].cpu().numpy(), ref, f"13B act-order qkv {name} S={s}")


# --------------------------------------------------- workload 4: 30B layer shapes, g=512
@pytest.mark.parametrize("k,n", [(6656, 6656), (17920, 6656)])
@pytest.mark.parametrize("m", [1, 8, 2048])
def test_30b_linear(k, n, m):
    g = 512
    L, W = layer_and_weights(k, n, g, 1400 + k // 128)
    D = to_dev(L)
    x = O.make_x(m, k, seed=1401 + m)
    xd = torch.from_numpy(x).cuda()
    y = gptq().matmul4(g, xd, D["qweight"], D["scales"], D["qzeros"])
    rows = sample_rows(m, 24, seed=n)
    assert_close(y[rows].cpu().numpy(), O.matmul_ref(x[rows], W), f"30B K={k} N={n} M={m}")
    if m > 16:
        p = torch.from_numpy(np.random.default_rng(10).permutation(m)).cuda()
        assert torch.equal(gptq().matmul4(g, xd[p], D["qweight"], D["scales"], D["qzeros"]), y[p])


@pytest.mark.parametrize("m", [1, 8, 2048])
def test_30b_mlp_gateup(m):
    k, n, g = 6656, 17920, 512
    (gate, Wg), (up, Wu) = layer_and_weights(k, n, g, 1410), layer_and_weights(k, n, g, 1411)
    Dg, Du = to_dev(gate), to_dev(up)
    x = O.make_x(m, k, seed=1412 + m)
    h = gptq().llama_mlp_4(g, torch.from_numpy(x).cuda(), Dg["qweight"], Dg["scales"], Dg["qzeros"],
                           Du["qweight"], Du["scales"], Du["qzeros"])
    rows = sample_rows(m, 16, seed=m + 3)
    ref = O.silu_mul_ref(O.matmul_ref(x[rows], Wg), O.matmul_ref(x[rows], Wu))
    assert_close(h[rows].cpu().numpy(), ref, f"30B gate/up M={m}")


@pytest.mark.parametrize("b,s,pos0", [(1, 1, 2047), (8, 1, 2047), (8, 256, 0)])
def test_30b_qkv_rotary(b, s, pos0):
    hidden, H, Dh, g = 6656, 52, 128, 512
    L = O.make_layer(hidden, 3 * hidden, g, seed=1420)
    D = to_dev(L)
    G = gptq()
    cos, sin = G.RotaryTable(Dh, 2304).get(torch.device("cuda"), 2304)
    x = O.make_x(b * s, hidden, seed=1421 + s).reshape(b, s, hidden)
    pos = (pos0 + np.arange(s, dtype=np.int64))[None, :].repeat(b, 0) + np.arange(b)[:, None]
    q, k, v = G.qkv_rotary(g, torch.from_numpy(x).cuda(), D["qweight"], D["scales"], D["qzeros"],
                           torch.from_numpy(pos).cuda(), cos, sin, H, Dh)
    rows = sample_rows(s, 6, seed=s)
    qr, kr, vr = O.qkv_rotary_ref(x[:, rows], L["qweight"], L["qzeros"], L["scales"], g, pos[:, rows], H, Dh,
                                  max_pos=2304)
    for got, ref, name in ((q, qr, "q"), (k, kr, "k"), (v, vr, "v")):
        assert got.shape == (b, H, s, Dh)
        assert_close(got[:, :, rows].cpu().numpy(), ref, f"30B qkv {name} b={b} s={s}")


# ------------------------------------------- workload 4 at its full batch: 8 sequences x 2048 tokens = 16384 rows
# The largest call any benchmark workload makes: 128 row tiles x 70 - 78 column panels of the tiled kernel, its banded
# tile order and the panels cut along K.  The oracle is evaluated on a sample of rows (first, last, tile boundaries,
# seeded); the rest is covered by the row-permutation property (bit-equal) and by one-hot rows (exact weight rows).
BIG = 16384


def big_rows(m, seed):
    fixed = [r for r in (0, 1, 127, 128, 129, 1023, 1024, 2047, 2048, 8191, 8192, m - 129, m - 128, m - 2, m - 1) if r < m]
    return np.unique(np.concatenate([np.array(fixed), np.random.default_rng(seed).choice(m, size=12, replace=False)]))


@pytest.mark.parametrize("k,n", [(6656, 6656), (17920, 6656)])
def test_30b_linear_at_16384_rows(k, n):
    g = 512
    L, W = layer_and_weights(k, n, g, 1400 + k // 128)
    D = to_dev(L)
    x = O.make_x(BIG, k, seed=1450)
    x[5] = 0
    x[5, 4321] = 1.0          # a one-hot row: the result is row 4321 of the weight, exactly
    xd = torch.from_numpy(x).cuda()
    y = gptq().matmul4(g, xd, D["qweight"], D["scales"], D["qzeros"])
    rows = big_rows(BIG, seed=n)
    assert_close(y[rows].cpu().numpy(), O.matmul_ref(x[rows], W), f"30B K={k} N={n} M={BIG}")
    assert (bits(y[5].cpu().numpy()) == bits(W[4321])).all()
    p = torch.from_numpy(np.random.default_rng(11).permutation(BIG)).cuda()
    assert torch.equal(gptq().matmul4(g, xd[p], D["qweight"], D["scales"], D["qzeros"]), y[p])


def test_30b_mlp_gateup_at_16384_rows():
    k, n, g = 6656, 17920, 512
    (gate, Wg), (up, Wu) = layer_and_weights(k, n, g, 1410), layer_and_weights(k, n, g, 1411)
    Dg, Du = to_dev(gate), to_dev(up)
    x = O.make_x(BIG, k, seed=1451)
    xd = torch.from_numpy(x).cuda()
    args = (Dg["qweight"], Dg["scales"], Dg["qzeros"], Du["qweight"], Du["scales"], Du["qzeros"])
    h = gptq().llama_mlp_4(g, xd, *args)
    rows = big_rows(BIG, seed=3)
    ref = O.silu_mul_ref(O.matmul_ref(x[rows], Wg), O.matmul_ref(x[rows], Wu))
    assert_close(h[rows].cpu().numpy(), ref, f"30B gate/up M={BIG}")
    p = torch.from_numpy(np.random.default_rng(12).permutation(BIG)).cuda()
    assert torch.equal(gptq().llama_mlp_4(g, xd[p], *args), h[p])


def test_30b_qkv_rotary_at_8_sequences_of_2048_tokens():
    hidden, H, Dh, g, b, s = 6656, 52, 128, 512, 8, 2048
    L = O.make_layer(hidden, 3 * hidden, g, seed=1420)
    D = to_dev(L)
    G = gptq()
    cos, sin = G.RotaryTable(Dh, 2304).get(torch.device("cuda"), 2304)
    x = O.make_x(b * s, hidden, seed=1452).reshape(b, s, hidden)
    pos = np.arange(s, dtype=np.int64)[None, :].repeat(b, 0) + np.arange(b)[:, None]
    xd, posd = torch.from_numpy(x).cuda(), torch.from_numpy(pos).cuda()
    q, k, v = G.qkv_rotary(g, xd, D["qweight"], D["scales"], D["qzeros"], posd, cos, sin, H, Dh)
    rows = np.array([0, 1, 127, 128, 1023, 1024, 2046, 2047])
    qr, kr, vr = O.qkv_rotary_ref(x[:, rows], L["qweight"], L["qzeros"], L["scales"], g, pos[:, rows], H, Dh, max_pos=2304)
    for got, ref, name in ((q, qr, "q"), (k, kr, "k"), (v, vr, "v")):
        assert got.shape == (b, H, s, Dh)
        assert_close(got[:, :, rows].cpu().numpy(), ref, f"30B qkv {name} b={b} s={s}")
    # the sequences in another order (positions go with them): the same bits, sequence by sequence
    p = torch.tensor([3, 0, 7, 1, 6, 2, 5, 4], device="cuda")
    q2, k2, v2 = G.qkv_rotary(g, xd[p].contiguous(), D["qweight"], D["scales"], D["qzeros"], posd[p].contiguous(), cos, sin, H, Dh)
    assert torch.equal(q2, q[p]) and torch.equal(k2, k[p]) and torch.equal(v2, v[p])


def test_7b_gate_up_at_8192_rows():
    k, n, g, m = 4096, 11008, 128, 8192
    (gate, Wg), (up, Wu) = layer_and_weights(k, n, g, 1460), layer_and_weights(k, n, g, 1461)
    Dg, Du = to_dev(gate), to_dev(up)
    x = O.make_x(m, k, seed=1462)
    xd = torch.from_numpy(x).cuda()
    args = (Dg["qweight"], Dg["scales"], Dg["qzeros"], Du["qweight"], Du["scales"], Du["qzeros"])
    h = gptq().llama_mlp_4(g, xd, *args)
    rows = big_rows(m, seed=4)
    ref = O.silu_mul_ref(O.matmul_ref(x[rows], Wg), O.matmul_ref(x[rows], Wu))
    assert_close(h[rows].cpu().numpy(), ref, f"7B gate/up M={m}")
    p = torch.from_numpy(np.random.default_rng(13).permutation(m)).cuda()
    assert torch.equal(gptq().llama_mlp_4(g, xd[p], *args), h[p])


# ------------------------------------------------------------- size-independent: one-hot rows
def test_one_hot_rows_at_full_size():
    """2048 one-hot rows through the 7B down_proj shape: every output row equals the
    dequantised weight row it selects, exactly (single term, no summation)."""
    k, n, g, m = 11008, 4096, 128, 2048
    L = O.make_layer(k, n, g, seed=1500)
    W = O.dequant_fp16(L["qweight"], L["qzeros"], L["scales"], g)
    sel = np.random.default_rng(1501).integers(0, k, size=m)
    x = np.zeros((m, k), dtype=np.float16)
    x[np.arange(m), sel] = 1.0
    D = to_dev(L)
    y = gptq().matmul4(g, torch.from_numpy(x).cuda(), D["qweight"], D["scales"], D["qzeros"])
    assert (bits(y.cpu().numpy()) == bits(W[sel])).all()


# ------------------------------------------------- derived copies follow in-place updates of the checkpoint tensors
def test_act_order_copies_follow_in_place_updates():
    """The sorted / column-ordered copies an act-order module derives at first use are keyed on the tensors'
    versions as well as their addresses: reloading weights into the existing buffers (load_state_dict, copy_)
    after a first forward must not keep serving the copies made from the old contents."""
    G = gptq()
    k, inter, g, m = 512, 768, 128, 3
    x = torch.from_numpy(O.make_x(m, k, seed=5)).cuda()

    def layers(seed):
        gate = O.make_layer(k, inter, g, seed=seed, act_order=True)
        up = O.make_layer(k, inter, g, seed=seed + 1)
        up["g_idx"] = gate["g_idx"]
        down = O.make_layer(inter, k, g, seed=seed + 2, act_order=True)
        return gate, up, down

    def build(seed):
        gate, up, down = layers(seed)
        return G.QuantLlamaMLP(quant_linear(gate, k, inter, g, True), quant_linear(down, inter, k, g, True),
                               quant_linear(up, k, inter, g, True)).cuda()

    old, new = build(100), build(200)
    y_old = old(x)
    want = new(x)
    assert not torch.equal(y_old, want)
    # the new weights into the OLD module's buffers, in place: same addresses, other contents
    old.load_state_dict(new.state_dict())
    assert torch.equal(old(x), want), "stale act-order copies served after an in-place reload"
    # a single QuantLinear likewise
    L1, L2 = O.make_layer(k, k, g, seed=300, act_order=True), O.make_layer(k, k, g, seed=301, act_order=True)
    a, b = quant_linear(L1, k, k, g, True).cuda(), quant_linear(L2, k, k, g, True).cuda()
    a(x)
    for name in ("qweight", "qzeros", "scales", "g_idx"):
        getattr(a, name).copy_(getattr(b, name))
    assert torch.equal(a(x), b(x))
