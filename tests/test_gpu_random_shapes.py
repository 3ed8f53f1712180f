"""GPU sweep over randomly drawn (rows, K, N) for the three fused operators with the automatic launch plans: which
kernel runs, its tile, K split, two launches over column ranges and strips shared along K all depend on how the tile
count of a shape relates to the CU count, and the fixed shapes of the other tests hit only some of those cases.

Checker: this library's own dequantised fp16 weights (bit-exact against the oracle, test_gpu_parity.py) multiplied in
float64 by torch on the GPU - wide accumulation on the canonical weights, which is what the oracle computes, at a size
the CPU oracle would take minutes for.  Same bars as test_gpu_parity.py.  A few draws are also checked against the
oracle itself."""
import numpy as np
import pytest
import torch

from conftest import to_dev
from oracle import gptq_oracle as O
from test_gpu_parity import ATOL, RTOL, gptq

pytestmark = pytest.mark.gpu


def close(y: torch.Tensor, ref: torch.Tensor, noise: torch.Tensor, what: str):
    """The stated tolerance, and a tight bound: half an fp16 step of the result plus `noise`, what fp32 accumulation may
    add before the rounding (see sum_noise)."""
    y = y.double()
    err = (y - ref).abs()
    assert bool((err <= ATOL + RTOL * ref.abs()).all()), f"{what}: max_abs={float(err.max()):.3e}"
    half = ref.abs().half()
    ulp = (torch.nextafter(half, torch.full_like(half, float("inf"))) - half).double()
    tight = 0.5 * ulp + noise + 1e-5 * ref.abs() + 1e-6
    assert bool((err <= tight).all()), f"{what}: {int((err > tight).sum())} elements beyond the tight bound, max_abs={float(err.max()):.3e}"


def sum_noise(x: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
    """Bound on the error of a dot product accumulated in fp32 in any order: a few fp32 roundings of the sum of the
    terms' magnitudes (2^-22 * |x| @ |W|; what the kernels show is a tenth of it).  It matters where a sum nearly
    cancels: relative to the result the error is then large, and a SiLU or a product carries it on."""
    return 2.0 ** -22 * (x.double().abs() @ w.abs())


def draw_shapes(seed: int, count: int, n_unit: int, n_max: int):
    rng = np.random.default_rng(seed)
    out = []
    for _ in range(count):
        m = int(np.exp(rng.uniform(0.0, np.log(4000))))
        k = 128 * int(rng.integers(2, 65))
        n = n_unit * int(rng.integers(1, n_max // n_unit + 1))
        groups = [g for g in (128, 256, 512, 1024) if k % g == 0] + [-1]
        g = groups[int(rng.integers(0, len(groups)))]
        out.append((m, k, n, g))
    return out


def layer(k, n, g, seed, bias=False):
    rng = np.random.default_rng(seed)
    groups = 1 if g == -1 else k // g
    L = {"qweight": rng.integers(-2**31, 2**31, size=(k // 8, n), dtype=np.int64).astype(np.int32),
         "qzeros": rng.integers(-2**31, 2**31, size=(groups, n // 8), dtype=np.int64).astype(np.int32),
         "scales": rng.uniform(0.002, 0.02, size=(groups, n)).astype(np.float16),
         "bias": rng.normal(0, 0.5, size=n).astype(np.float16) if bias else None}
    return L


def dequant64(G, D, k, g):
    return G.dequantize(D["qweight"], D["qzeros"], D["scales"], k if g == -1 else g, None).double()


@pytest.mark.parametrize("m,k,n,g", draw_shapes(1, 200, 256, 16384))
def test_plain_projection(m, k, n, g):
    G = gptq()
    L = layer(k, n, g, seed=m + k + n, bias=(m % 3 == 0))
    D = to_dev(L)
    x = torch.from_numpy(O.make_x(m, k, seed=m)).cuda()
    y = G.matmul4(k if g == -1 else g, x, D["qweight"], D["scales"], D["qzeros"], D.get("bias"))
    w = dequant64(G, D, k, g)
    ref = x.double() @ w
    if L["bias"] is not None:
        # the kernels add the bias to the rounded fp16 product, as the reference's module does
        ref = (ref.half() + D["bias"]).double()
        err = (y.double() - ref).abs()
        assert bool((err <= ATOL + RTOL * ref.abs()).all()), f"M={m} K={k} N={n} g={g}: max_abs={float(err.max()):.3e}"
    else:
        close(y, ref, sum_noise(x, w), f"matmul M={m} K={k} N={n} g={g}")


@pytest.mark.parametrize("m,k,n,g", draw_shapes(2, 150, 256, 14336))
def test_gate_up(m, k, n, g):
    G = gptq()
    Dg, Du = to_dev(layer(k, n, g, seed=m + n)), to_dev(layer(k, n, g, seed=m + n + 1))
    x = torch.from_numpy(O.make_x(m, k, seed=m)).cuda()
    gs = k if g == -1 else g
    h = G.llama_mlp_4(gs, x, Dg["qweight"], Dg["scales"], Dg["qzeros"], Du["qweight"], Du["scales"], Du["qzeros"])
    wg, wu = dequant64(G, Dg, k, g), dequant64(G, Du, k, g)
    a, b = x.double() @ wg, x.double() @ wu
    silu = a / (1.0 + torch.exp(-a))
    ref = silu * b
    # |d silu / da| <= 1.1
    close(h, ref, 1.1 * b.abs() * sum_noise(x, wg) + silu.abs() * sum_noise(x, wu), f"gate/up M={m} K={k} N={n} g={g}")


@pytest.mark.parametrize("m,k,n,g", draw_shapes(3, 150, 768, 19968))
def test_qkv_rotary(m, k, n, g):
    """n = 3 * heads * 128 with an even number of heads (N is a multiple of 256); positions scattered over the table."""
    G = gptq()
    heads = n // 384
    D = to_dev(layer(k, n, g, seed=m + n + 2))
    x = torch.from_numpy(O.make_x(m, k, seed=m + 1)).cuda()
    rng = np.random.default_rng(m)
    pos = torch.from_numpy(rng.integers(0, 4096, size=(1, m)).astype(np.int32)).cuda()
    cos, sin = G.RotaryTable(128, 4096).get(torch.device("cuda"), 4096)
    q, kk, v = G.qkv_rotary(k if g == -1 else g, x.view(1, m, k), D["qweight"], D["scales"], D["qzeros"], pos, cos, sin, heads)
    w = dequant64(G, D, k, g)
    y = (x.double() @ w).view(m, 3, heads, 128)
    noise = sum_noise(x, w).view(m, 3, heads, 128)
    swapped = torch.cat([noise[..., 64:], noise[..., :64]], dim=-1)  # a rotated value mixes columns d and d +- 64
    c, s = cos[pos[0].long()].double(), sin[pos[0].long()].double()          # [m, 64]

    def rotate(t):   # [m, heads, 128]
        lo, hi = t[..., :64], t[..., 64:]
        return torch.cat([lo * c[:, None] - hi * s[:, None], hi * c[:, None] + lo * s[:, None]], dim=-1)

    for i, (got, ref, name) in enumerate(((q, rotate(y[:, 0]), "q"), (kk, rotate(y[:, 1]), "k"), (v, y[:, 2], "v"))):
        close(got[0].transpose(0, 1), ref, noise[:, i] + (swapped[:, i] if i < 2 else 0.0), f"{name} M={m} K={k} heads={heads} g={g}")


@pytest.mark.parametrize("idx", [0, 7, 19])
def test_the_checker_agrees_with_the_oracle(idx):
    """The float64 product of the dequantised weights is the oracle's reference: compared directly on draws small
    enough for the CPU."""
    G = gptq()
    shapes = [s for s in draw_shapes(1, 200, 256, 16384) if 1e8 < s[0] * s[1] * s[2] < 3e9]
    m, k, n, g = shapes[idx % len(shapes)]
    L = layer(k, n, g, seed=m + k + n)
    D = to_dev(L)
    x = O.make_x(m, k, seed=m)
    ref = O.quant_matmul_ref(x, L["qweight"], L["qzeros"], L["scales"], g)
    mine = (torch.from_numpy(x).cuda().double() @ dequant64(G, D, k, g)).cpu().numpy()
    # (the oracle hands its float64 sums back rounded to float32)
    assert (np.abs(mine - ref) <= 2.0 ** -23 * np.abs(ref) + 1e-9).all()


@pytest.mark.parametrize("m,k,n,g", [s for s in draw_shapes(4, 90, 256, 8192) if s[3] != -1][:60])
def test_act_order_projection(m, k, n, g):
    """Rows of the weight in a random group order (g_idx): the sorted copy and the permutation made at load time, the
    activations gathered by the call; plain projection and the gate/up pair on the same draw."""
    G = gptq()
    rng = np.random.default_rng(m + k)
    g_idx = torch.from_numpy(rng.permutation(np.repeat(np.arange(k // g), g)).astype(np.int32)).cuda()
    Dg, Du = to_dev(layer(k, n, g, seed=m + n + 5)), to_dev(layer(k, n, g, seed=m + n + 6))
    x = torch.from_numpy(O.make_x(m, k, seed=m + 2)).cuda()
    wg = G.dequantize(Dg["qweight"], Dg["qzeros"], Dg["scales"], g, g_idx).double()
    wu = G.dequantize(Du["qweight"], Du["qzeros"], Du["scales"], g, g_idx).double()
    gq, perm = G.prepare_act_order(Dg["qweight"], g_idx, g)
    uq, _ = G.prepare_act_order(Du["qweight"], g_idx, g)
    y = G.matmul4(g, x, gq, Dg["scales"], Dg["qzeros"], None, perm)
    close(y, x.double() @ wg, sum_noise(x, wg), f"act-order matmul M={m} K={k} N={n} g={g}")
    h = G.llama_mlp_4(g, x, gq, Dg["scales"], Dg["qzeros"], uq, Du["scales"], Du["qzeros"], perm=perm)
    a, b = x.double() @ wg, x.double() @ wu
    silu = a / (1.0 + torch.exp(-a))
    close(h, silu * b, 1.1 * b.abs() * sum_noise(x, wg) + silu.abs() * sum_noise(x, wu), f"act-order gate/up M={m} K={k} N={n} g={g}")


@pytest.mark.parametrize("m,k,n", [(3400, 2048, 2560), (700, 4096, 6144), (1300, 2048, 5632)])
def test_act_order_gathered_by_the_tiled_kernel_itself_with_shared_panels(m, k, n):
    """The tiled kernel's own act-order gather (what calls too large to stage use; forced here) on tile counts just above
    a whole number of rounds, where the last column panels are cut along K inside the launch: plain projection and the
    gate/up pair."""
    from gptq_triton_amd import _lib
    lib = _lib.load()
    G = gptq()
    g = 128
    rng = np.random.default_rng(m)
    g_idx = torch.from_numpy(rng.permutation(np.repeat(np.arange(k // g), g)).astype(np.int32)).cuda()
    Dg, Du = to_dev(layer(k, n, g, seed=m + 7)), to_dev(layer(k, n, g, seed=m + 8))
    x = torch.from_numpy(O.make_x(m, k, seed=m + 3)).cuda()
    wg = G.dequantize(Dg["qweight"], Dg["qzeros"], Dg["scales"], g, g_idx).double()
    wu = G.dequantize(Du["qweight"], Du["qzeros"], Du["scales"], g, g_idx).double()
    gq, perm = G.prepare_act_order(Dg["qweight"], g_idx, g)
    uq, _ = G.prepare_act_order(Du["qweight"], g_idx, g)
    try:
        lib.gptq4_set_midm_tuning(0, 0, 0)
        lib.gptq4_set_gemm_tuning(10, 0)
        y = G.matmul4(g, x, gq, Dg["scales"], Dg["qzeros"], None, perm)
        h = G.llama_mlp_4(g, x, gq, Dg["scales"], Dg["qzeros"], uq, Du["scales"], Du["qzeros"], perm=perm)
    finally:
        lib.gptq4_set_gemm_tuning(0, 0)
        lib.gptq4_set_midm_tuning(1, 0, 0)
    close(y, x.double() @ wg, sum_noise(x, wg), f"own gather, matmul M={m} K={k} N={n}")
    a, b = x.double() @ wg, x.double() @ wu
    silu = a / (1.0 + torch.exp(-a))
    close(h, silu * b, 1.1 * b.abs() * sum_noise(x, wg) + silu.abs() * sum_noise(x, wu), f"own gather, gate/up M={m} K={k} N={n}")
