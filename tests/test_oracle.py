"""Pins for the CPU oracle (oracle/gptq_oracle.py), CPU only.

The reference holds no golden vectors for this path (its checks live in a GPU-only
notebook and record only max-abs differences), so the oracle is pinned against what
the mathematics fixes: bit-by-bit brute force on tiny inputs, exhaustive enumeration
with exact rational arithmetic, library routines, closed forms and invariants.  Each
check is chosen so that a plausible mistake - a shifted nibble, swapped axes, a
missing "+1" on the zero, a double rounding, a wrong rotary sign - fails it.
"""
from fractions import Fraction

import numpy as np
import pytest

from conftest import bits
from oracle import brute
from oracle import gptq_oracle as O


# ----------------------------------------------------------------------- bit layout
def test_unpack_known_words():
    # field t of the word holds row 8r+t: 0x76543210 -> rows 0..7 = 0..7
    qw = np.array([[0x76543210, -1, 0, np.int32(-2**31)]], dtype=np.int64).astype(np.int32)
    q = O.unpack_qweight(qw)
    assert q[:, 0].tolist() == [0, 1, 2, 3, 4, 5, 6, 7]
    assert q[:, 1].tolist() == [15] * 8            # 0xFFFFFFFF: sign fill must be masked off
    assert q[:, 2].tolist() == [0] * 8
    assert q[:, 3].tolist() == [0] * 7 + [8]       # only the sign bit set -> top nibble = 8
    qz = np.array([[0x76543210, np.int32(-2**31)]], dtype=np.int64).astype(np.int32)
    z = O.unpack_qzeros(qz)
    assert z[0].tolist() == [0, 1, 2, 3, 4, 5, 6, 7] + [0] * 7 + [8]   # field t -> column 8c+t


def test_unpack_matches_bit_loops():
    rng = np.random.default_rng(0)
    qw = rng.integers(-2**31, 2**31, size=(2, 8), dtype=np.int64).astype(np.int32)   # K=16, N=8
    qz = rng.integers(-2**31, 2**31, size=(2, 1), dtype=np.int64).astype(np.int32)
    assert O.unpack_qweight(qw).tolist() == brute.unpack_qweight_loops(qw.tolist())
    assert O.unpack_qzeros(qz).tolist() == brute.unpack_qzeros_loops(qz.tolist())


def test_pack_unpack_round_trip():
    rng = np.random.default_rng(1)
    q = rng.integers(0, 16, size=(64, 24), dtype=np.uint8)
    z = rng.integers(0, 16, size=(4, 24), dtype=np.uint8)
    assert (O.unpack_qweight(O.pack_qweight(q)) == q).all()
    assert (O.unpack_qzeros(O.pack_qzeros(z)) == z).all()
    w = rng.integers(-2**31, 2**31, size=(8, 24), dtype=np.int64).astype(np.int32)
    assert (O.pack_qweight(O.unpack_qweight(w)) == w).all()
    # the packers themselves against the definition, element by element
    pw = O.pack_qweight(q)
    for (k, n) in [(0, 0), (7, 3), (8, 3), (63, 23), (13, 5)]:
        assert brute.nibble(int(pw[k // 8, n]), k % 8) == q[k, n]
    pz = O.pack_qzeros(z)
    for (g, n) in [(0, 0), (3, 23), (1, 8), (2, 15)]:
        assert brute.nibble(int(pz[g, n // 8]), n % 8) == z[g, n]


# -------------------------------------------------------------------------- dequant
def test_dequant_exhaustive_against_exact_rationals():
    """All 16 x 16 (q, z) pairs x every fp16 scale in [0.002, 0.02] (3,3xx values):
    the oracle must equal the exact product rounded once to fp16."""
    lo, hi = np.float16(0.002).view(np.uint16), np.float16(0.02).view(np.uint16)
    s_vals = np.arange(lo, hi + 1, dtype=np.uint16).view(np.float16)
    assert len(s_vals) > 3000
    n = len(s_vals) * 16
    scales = np.repeat(s_vals, 16)[None, :]
    z = np.tile(np.arange(16, dtype=np.uint8), len(s_vals))[None, :]
    q = np.tile(np.arange(16, dtype=np.uint8)[:, None], (1, n))
    W = O.dequant_fp16(O.pack_qweight(q), O.pack_qzeros(z), scales, -1)
    # exact: (q - z - 1) * s as a rational, one rounding to fp16
    s64 = scales.astype(np.float64)   # fp16 -> float64 is exact
    d = q.astype(np.int64) - (z.astype(np.int64) + 1)
    exact = d.astype(np.float64) * s64   # |d| <= 16 and s has 11 significant bits: exact in float64
    assert (bits(W) == bits(exact.astype(np.float16))).all()
    # spot-check the float64 shortcut itself with true rationals
    for (i, j) in [(0, 0), (15, 17), (3, n - 1), (9, 12345), (0, 15)]:
        fr = Fraction(int(d[i, j])) * Fraction(float(scales[0, j]))
        assert bits(W[i, j]) == bits(brute.fp16_round(fr))
    # q = z + 1 decodes to +0 (not -0)
    assert bits(W[1, 0]) == 0 and d[1, 0] == 0


def test_dequant_matches_loops_with_groups_and_g_idx():
    L = O.make_layer(32, 16, 16, seed=3, act_order=True)
    for g_idx in (None, L["g_idx"]):
        W = O.dequant_fp16(L["qweight"], L["qzeros"], L["scales"], 16, g_idx)
        Wb = brute.dequant_loops(L["qweight"].tolist(), L["qzeros"].tolist(), L["scales"], 16, g_idx)
        assert (bits(W) == bits(Wb)).all()
    L1 = O.make_layer(16, 8, -1, seed=4)
    W = O.dequant_fp16(L1["qweight"], L1["qzeros"], L1["scales"], -1)
    Wb = brute.dequant_loops(L1["qweight"].tolist(), L1["qzeros"].tolist(), L1["scales"], -1)
    assert (bits(W) == bits(Wb)).all()


def test_trivial_g_idx_is_identity_and_permuted_is_gather():
    k, n, g = 256, 16, 64
    L = O.make_layer(k, n, g, seed=5, act_order=True)
    base = O.dequant_fp16(L["qweight"], L["qzeros"], L["scales"], g)
    same = O.dequant_fp16(L["qweight"], L["qzeros"], L["scales"], g, np.arange(k) // g)
    assert (bits(base) == bits(same)).all()
    W = O.dequant_fp16(L["qweight"], L["qzeros"], L["scales"], g, L["g_idx"])
    q = O.unpack_qweight(L["qweight"]).astype(np.float32)
    z = O.unpack_qzeros(L["qzeros"]).astype(np.float32)
    for kk in (0, 1, 100, 255):
        gi = int(L["g_idx"][kk])
        row = ((q[kk] - z[gi] - 1) * L["scales"][gi].astype(np.float32)).astype(np.float16)
        assert (bits(W[kk]) == bits(row)).all()


def test_triton_rounding_order_differs_from_canonical():
    """Documents why 'bit-exact' needs ONE stated order: the reference kernel's own
    three-rounding order is not the README formula's single rounding."""
    L = O.make_layer(1024, 64, -1, seed=6)
    a = O.dequant_fp16(L["qweight"], L["qzeros"], L["scales"], -1)
    b = O.dequant_triton_order(L["qweight"], L["qzeros"], L["scales"], -1)
    frac = (bits(a) != bits(b)).mean()
    assert 0.2 < frac < 0.7
    assert np.abs(a.astype(np.float32) - b.astype(np.float32)).max() < 3e-4


# --------------------------------------------------------------------------- matmul
def test_matmul_against_exact_rationals_tiny():
    L = O.make_layer(16, 8, 8, seed=7)
    x = O.make_x(3, 16, seed=8)
    W = O.dequant_fp16(L["qweight"], L["qzeros"], L["scales"], 8)
    y = O.quant_matmul_ref(x, L["qweight"], L["qzeros"], L["scales"], 8)
    exact = brute.matmul_loops(x.tolist(), W.tolist())
    assert np.abs(y - exact).max() <= 1e-6 * max(1.0, np.abs(exact).max())


def test_matmul_invariants():
    k, n, g = 512, 64, 128
    L = O.make_layer(k, n, g, seed=9, bias=True)
    W = O.dequant_fp16(L["qweight"], L["qzeros"], L["scales"], g)
    x1, x2 = O.make_x(4, k, 10), O.make_x(4, k, 11)
    f = lambda x, **kw: O.quant_matmul_ref(x, L["qweight"], L["qzeros"], L["scales"], g, **kw)
    # zero input -> zero (+ bias)
    assert (f(np.zeros((2, k), np.float16)) == 0).all()
    assert np.allclose(f(np.zeros((2, k), np.float16), bias=L["bias"]), L["bias"].astype(np.float32))
    # one-hot input -> that row of W, exactly
    e = np.zeros((1, k), np.float16)
    e[0, 137] = 1
    assert (f(e)[0] == W[137].astype(np.float32)).all()
    # linearity (x1 + x2 formed in float64 to stay exact)
    lhs = (x1.astype(np.float64) + x2.astype(np.float64)) @ W.astype(np.float64)
    assert np.allclose(lhs, f(x1).astype(np.float64) + f(x2), atol=1e-4)
    # column independence: a column slice computed alone has identical bits
    sl = slice(16, 40)
    Ls = dict(qweight=L["qweight"][:, sl], qzeros=L["qzeros"][:, 2:5], scales=L["scales"][:, sl])
    ys = O.quant_matmul_ref(x1, Ls["qweight"], Ls["qzeros"], Ls["scales"], g)
    assert (ys == f(x1)[:, sl]).all()
    # batch dims are flattened and restored
    x3 = np.stack([x1, x2])
    assert f(x3).shape == (2, 4, n) and (f(x3)[1] == f(x2)).all()


def test_numpy_and_torch_cpu_baseline_agree():
    import torch
    from oracle import torch_cpu as T
    k, n, g = 1024, 256, 128
    L = O.make_layer(k, n, g, seed=12, act_order=True, bias=True)
    x = O.make_x(5, k, 13)
    t = {key: torch.from_numpy(v) for key, v in L.items() if isinstance(v, np.ndarray)}
    Wt = T.dequant_fp16(t["qweight"], t["qzeros"], t["scales"], g, t["g_idx"])
    Wn = O.dequant_fp16(L["qweight"], L["qzeros"], L["scales"], g, L["g_idx"])
    assert (bits(Wt.numpy()) == bits(Wn)).all()
    yt = T.quant_matmul(torch.from_numpy(x), t["qweight"], t["qzeros"], t["scales"], g, t["bias"], t["g_idx"])
    yn = O.quant_matmul_ref(x, L["qweight"], L["qzeros"], L["scales"], g, bias=L["bias"], g_idx=L["g_idx"])
    assert np.abs(yt.numpy() - yn).max() < 1e-4


# ------------------------------------------------------------------------------ MLP
def test_silu_known_values_and_identity():
    x = np.array([0.0, 1.0, -1.0, 20.0, -20.0, 0.5], dtype=np.float64)
    s = O.silu(x)
    assert s[0] == 0.0
    assert abs(s[1] - 0.7310585786300049) < 1e-15 and abs(s[2] + 0.2689414213699951) < 1e-15
    assert abs(s[3] - 20.0) < 1e-7 and abs(s[4]) < 1e-7
    # x*sigmoid(x) == x/2 * (1 + tanh(x/2))
    xs = np.linspace(-12, 12, 1001)
    assert np.allclose(O.silu(xs), xs / 2 * (1 + np.tanh(xs / 2)), atol=1e-12)
    # the gate gets the SiLU, not the up projection
    assert np.allclose(O.silu_mul_ref(np.array([1.0]), np.array([3.0])), 3 * 0.7310585786300049)
    assert not np.allclose(O.silu_mul_ref(np.array([1.0]), np.array([3.0])),
                           O.silu_mul_ref(np.array([3.0]), np.array([1.0])))


def test_mlp_composition():
    k, i, g = 256, 512, 128
    gate, up, down = (O.make_layer(k, i, g, 20), O.make_layer(k, i, g, 21), O.make_layer(i, k, g, 22))
    trip = lambda L: (L["qweight"], L["qzeros"], L["scales"])
    x = O.make_x(3, k, 23)
    h = O.mlp_gateup_ref(x, trip(gate), trip(up), g)
    a = O.quant_matmul_ref(x, *trip(gate), g).astype(np.float64)
    b = O.quant_matmul_ref(x, *trip(up), g).astype(np.float64)
    assert np.allclose(h, a / (1 + np.exp(-a)) * b, rtol=1e-6)
    y = O.mlp_ref(x, trip(gate), trip(up), trip(down), g)
    assert np.allclose(y, O.quant_matmul_ref(h.astype(np.float16), *trip(down), g))


# --------------------------------------------------------------------------- rotary
def test_rotary_tables_closed_form():
    cos, sin = O.rotary_tables(2048, 128, 10000.0)
    assert cos.shape == (2048, 64) and cos.dtype == np.float32
    assert (cos[0] == 1).all() and (sin[0] == 0).all()              # p = 0: identity
    assert abs(cos[1, 0] - np.cos(1.0)) < 1e-7 and abs(sin[1, 0] - np.sin(1.0)) < 1e-7   # inv_freq[0] = 1
    # inv_freq[i] = 10000^(-i/64): i = 32 -> 1/100
    assert abs(cos[100, 32] - np.cos(1.0)) < 1e-6 and abs(sin[50, 32] - np.sin(0.5)) < 1e-6
    assert np.abs(cos ** 2 + sin ** 2 - 1).max() < 1e-6


def test_rotary_properties():
    rng = np.random.default_rng(30)
    cos, sin = O.rotary_tables(512, 128)
    c64, s64 = cos.astype(np.float64), sin.astype(np.float64)
    x = rng.standard_normal((5, 128))
    # identity at p = 0
    assert np.allclose(O.apply_rotary(x, cos[0], sin[0]), x)
    # each (d, d+64) pair is rotated: norms preserved
    y = O.apply_rotary(x, cos[17], sin[17])
    assert np.allclose(x[:, :64] ** 2 + x[:, 64:] ** 2, y[:, :64] ** 2 + y[:, 64:] ** 2)
    # sign convention: the first half gets  x1*cos - x2*sin
    e = np.zeros(128)
    e[64] = 1.0                                         # x2 = 1 at d = 0
    r = O.apply_rotary(e, cos[1], sin[1])
    assert abs(r[0] + np.sin(1.0)) < 1e-6 and abs(r[64] - np.cos(1.0)) < 1e-6
    # composition R(p1) R(p2) = R(p1 + p2) (exact angles, so use inv_freq-exact pairs)
    exact = lambda p: (np.cos(p * (1.0 / 10000 ** (np.arange(64) / 64))), np.sin(p * (1.0 / 10000 ** (np.arange(64) / 64))))
    a = O.apply_rotary(O.apply_rotary(x, *exact(3)), *exact(9))
    assert np.allclose(a, O.apply_rotary(x, *exact(12)))
    # relative-position property of the inner product
    q, k = rng.standard_normal(128), rng.standard_normal(128)
    d1 = O.apply_rotary(q, c64[40], s64[40]) @ O.apply_rotary(k, c64[10], s64[10])
    d2 = O.apply_rotary(q, c64[130], s64[130]) @ O.apply_rotary(k, c64[100], s64[100])
    assert abs(d1 - d2) < 1e-3
    # the fp16-order variant (reference-era rounding) stays within a few fp16 ulps
    x16 = x.astype(np.float16)
    ex = O.apply_rotary(x16, cos[300], sin[300])
    lo = O.apply_rotary_fp16_order(x16, cos[300], sin[300]).astype(np.float64)
    assert np.abs(lo - ex).max() < 4e-3


def test_qkv_rotary_layout():
    H, Dh, hidden, g = 2, 128, 256, 128
    L = O.make_layer(hidden, 3 * hidden, g, seed=31)
    x = O.make_x(6, hidden, 32).reshape(2, 3, hidden)
    pos = np.array([[5, 6, 7], [0, 1, 2]])
    q, k, v = O.qkv_rotary_ref(x, L["qweight"], L["qzeros"], L["scales"], g, pos, H, Dh)
    y = O.quant_matmul_ref(x, L["qweight"], L["qzeros"], L["scales"], g)
    assert q.shape == (2, H, 3, Dh)
    # v is column block [2h, 3h), head-major, untouched
    assert (v[1, 1, 2] == y[1, 2, 2 * hidden + Dh:2 * hidden + 2 * Dh]).all()
    # position 0 leaves q and k as projected
    assert np.allclose(q[1, 0, 0], y[1, 0, 0:Dh]) and np.allclose(k[1, 1, 0], y[1, 0, hidden + Dh:hidden + 2 * Dh])
    # a rotated row equals the closed form on the projected row
    cos, sin = O.rotary_tables(8, Dh)
    assert np.allclose(k[0, 1, 2], O.apply_rotary(y[0, 2, hidden + Dh:hidden + 2 * Dh], cos[7], sin[7]), atol=1e-5)


# ------------------------------------------------------------------ decoder-side operators
def test_rmsnorm_oracle_special_cases():
    rng = np.random.default_rng(0)
    w = rng.standard_normal(64).astype(np.float16)
    # a constant row normalises to +-1 exactly, so y = +-weight
    for c in (3.0, -0.25):
        y = O.rmsnorm_ref(np.full((2, 64), c, dtype=np.float16), w, 0.0)
        assert (y == np.sign(c).astype(np.float16) * w).all()
    # invariant under scaling of x when eps = 0 (powers of two keep fp16 inputs exact)
    x = rng.standard_normal((3, 64)).astype(np.float16)
    assert (O.rmsnorm_ref(x, w, 0.0) == O.rmsnorm_ref(x * np.float16(4.0), w, 0.0)).all()
    # unit weight: the output row has mean square 1 up to fp16 rounding
    y = O.rmsnorm_ref(x, np.ones(64, dtype=np.float16), 1e-6).astype(np.float64)
    assert np.allclose((y * y).mean(-1), 1.0, atol=2e-3)
    # eps matters for tiny rows: x = 0 gives 0, not NaN
    assert (O.rmsnorm_ref(np.zeros((1, 64), dtype=np.float16), w, 1e-6) == 0).all()


def test_decode_attention_oracle_special_cases():
    rng = np.random.default_rng(1)
    B, H, cap, D = 2, 3, 9, 128
    q = rng.standard_normal((B, H, 1, D)).astype(np.float16)
    k = rng.standard_normal((B, H, cap, D)).astype(np.float16)
    v = rng.standard_normal((B, H, cap, D)).astype(np.float16)
    # position 0: the only visible row
    out = O.decode_attention_ref(q, k, v, [0, 0])
    assert np.array_equal(out.reshape(B, H, D), v[:, :, 0].astype(np.float64))
    # equal keys: uniform weights, the mean of the visible V rows
    k_eq = np.broadcast_to(k[:, :, :1], k.shape)
    out = O.decode_attention_ref(q, k_eq, v, [4, 8])
    assert np.allclose(out[0].reshape(H, D), v[0, :, :5].astype(np.float64).mean(1))
    assert np.allclose(out[1].reshape(H, D), v[1, :, :9].astype(np.float64).mean(1))
    # one key aligned with a large query dominates: its V row comes out
    qb = np.zeros((1, 1, 1, D), dtype=np.float16); qb[..., 0] = 200.0
    kb = np.zeros((1, 1, cap, D), dtype=np.float16); kb[0, 0, 6, 0] = 10.0
    out = O.decode_attention_ref(qb, kb, v[:1, :1], [8])
    assert np.allclose(out.reshape(D), v[0, 0, 6].astype(np.float64), atol=1e-9)
    # rows beyond the position are invisible
    v2 = v.copy(); v2[:, :, 5:] = 1e4
    assert np.array_equal(O.decode_attention_ref(q, k, v, [4, 4]), O.decode_attention_ref(q, k, v2, [4, 4]))


def test_prefill_attention_ref_is_the_single_query_form_row_by_row_and_torchs_causal_attention():
    import torch
    rng = np.random.default_rng(7)
    b, h, s, past, d = 2, 3, 9, 4, 128
    q = rng.standard_normal((b, h, s, d)).astype(np.float16)
    k = rng.standard_normal((b, h, past + s + 2, d)).astype(np.float16)
    v = rng.standard_normal((b, h, past + s + 2, d)).astype(np.float16)
    out = O.prefill_attention_ref(q, k, v, past)
    for i in range(s):
        one = O.decode_attention_ref(q[:, :, i:i + 1], k, v, [past + i] * b)
        assert np.allclose(out[:, i], one[:, 0], rtol=0, atol=1e-12)
    # no past: the library routine with its own causal mask
    out0 = O.prefill_attention_ref(q, k, v, 0)
    tq, tk, tv = (torch.from_numpy(a.astype(np.float64)) for a in (q, k[:, :, :s], v[:, :, :s]))
    ref = torch.nn.functional.scaled_dot_product_attention(tq, tk, tv, is_causal=True).transpose(1, 2).reshape(b, s, h * d)
    assert np.allclose(out0, ref.numpy(), rtol=0, atol=1e-10)
