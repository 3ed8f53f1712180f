"""CPU oracle for the 4-bit GPTQ inference hot path.  TEST INFRASTRUCTURE ONLY.

This module is the checker, never the product: only tests/, __graft_entry__.smoke()
and bench.py's cpu_baseline leg may import it.  The product path (the HIP library
behind gptq_triton_amd) never calls anything in here.

It restates, in numpy, the arithmetic of the reference hot path.  Every function
cites the reference lines it follows (paths relative to the reference checkout).

How each function is pinned (the reference ships no golden vectors, only tolerance
bands in Verify.ipynb, so the pins are mathematical):

  unpack_qweight / unpack_qzeros   brute-force bit loops (oracle/brute.py) on tiny
                                   tensors, sign-bit / all-ones / all-zero words,
                                   unpack(pack(q)) == q round trip.
  pack_qweight / pack_qzeros       round trip with the unpackers + brute force.
  dequant_fp16                     exhaustive enumeration of all 16x16 (q, z) pairs
                                   times every fp16 scale in [0.002, 0.02] against
                                   exact rational arithmetic (fractions.Fraction)
                                   rounded once to fp16.
  matmul_ref                       reduces to a library routine (float64 matmul on the
                                   dequantised weights); linearity, one-hot rows,
                                   column independence.
  silu_mul_ref                     textbook x*sigmoid(x), checked against the
                                   exp-free tanh identity and known values.
  rotary_tables / apply_rotary     closed form; p=0 identity, norm preservation,
                                   R(p1)R(p2)=R(p1+p2), relative-position property.
                                   PARITY UNPINNED BY THE REFERENCE: the reference
                                   delegates rotary to an unvendored third-party
                                   package (transformers, unpinned in setup.cfg:33)
                                   and its own check (Verify.ipynb:167-217) compares
                                   two paths through that same code.  The closed form
                                   restated here is the published GPT-NeoX
                                   "rotate_half" convention that package implements.
  g_idx handling                   g_idx = arange(K)//groupsize reproduces the
                                   un-indexed result bit for bit; a permuted g_idx
                                   equals an explicit per-row gather.
"""
from __future__ import annotations

import numpy as np

NIBBLES_PER_WORD = 8


# --------------------------------------------------------------------------- format
def unpack_qweight(qweight: np.ndarray) -> np.ndarray:
    """int32 [K/8, N] -> uint8 [K, N].

    Bits [4t, 4t+4) of qweight[r, n] hold the nibble of input row k = 8r + t
    (quantize.py:262-271 packs `intweight[j] << (bits * (j - i))`; the kernel
    decodes with `(b >> ((offs_k % 8) * 4)) & 0xF`, quant_linear.py:171,177,211).
    The shift is arithmetic on a signed word; the mask removes the sign fill.
    """
    qweight = np.ascontiguousarray(qweight, dtype=np.int32)
    rows, n = qweight.shape
    u = qweight.view(np.uint32)
    out = np.empty((rows, NIBBLES_PER_WORD, n), dtype=np.uint8)
    for t in range(NIBBLES_PER_WORD):
        out[:, t, :] = (u >> np.uint32(4 * t)) & np.uint32(0xF)
    return out.reshape(rows * NIBBLES_PER_WORD, n)


def unpack_qzeros(qzeros: np.ndarray) -> np.ndarray:
    """int32 [G, N/8] -> uint8 [G, N] of STORED zeros (true zero minus one).

    Bits [4t, 4t+4) of qzeros[g, c] belong to output column n = 8c + t
    (quantize.py:276-289; decoded at quant_linear.py:178,187 with
    `(zeros >> ((offs_bn % 8) * 4)) & 0xF`).
    """
    qzeros = np.ascontiguousarray(qzeros, dtype=np.int32)
    g, c = qzeros.shape
    u = qzeros.view(np.uint32)
    out = np.empty((g, c, NIBBLES_PER_WORD), dtype=np.uint8)
    for t in range(NIBBLES_PER_WORD):
        out[:, :, t] = (u >> np.uint32(4 * t)) & np.uint32(0xF)
    return out.reshape(g, c * NIBBLES_PER_WORD)


def pack_qweight(q: np.ndarray) -> np.ndarray:
    """uint8 nibbles [K, N] -> int32 [K/8, N]; inverse of unpack_qweight
    (restates the OR-shift loop of quantize.py:262-271)."""
    q = np.asarray(q)
    k, n = q.shape
    assert k % NIBBLES_PER_WORD == 0
    assert q.min(initial=0) >= 0 and q.max(initial=0) <= 15
    w = np.zeros((k // NIBBLES_PER_WORD, n), dtype=np.uint32)
    q3 = q.reshape(k // NIBBLES_PER_WORD, NIBBLES_PER_WORD, n).astype(np.uint32)
    for t in range(NIBBLES_PER_WORD):
        w |= q3[:, t, :] << np.uint32(4 * t)
    return w.view(np.int32)


def pack_qzeros(z_stored: np.ndarray) -> np.ndarray:
    """uint8 stored zeros [G, N] -> int32 [G, N/8]; inverse of unpack_qzeros
    (restates quantize.py:276-289; the caller has already subtracted one)."""
    z = np.asarray(z_stored)
    g, n = z.shape
    assert n % NIBBLES_PER_WORD == 0
    assert z.min(initial=0) >= 0 and z.max(initial=0) <= 15
    w = np.zeros((g, n // NIBBLES_PER_WORD), dtype=np.uint32)
    z3 = z.reshape(g, n // NIBBLES_PER_WORD, NIBBLES_PER_WORD).astype(np.uint32)
    for t in range(NIBBLES_PER_WORD):
        w |= z3[:, :, t] << np.uint32(4 * t)
    return w.view(np.int32)


def group_index(k: int, groupsize: int, g_idx: np.ndarray | None = None) -> np.ndarray:
    """Group of every input row: g_idx if given, else k // groupsize
    (quantize.py:253; README.md:95).  groupsize == -1 means one group."""
    if groupsize == -1:
        groupsize = k
    if g_idx is not None:
        g = np.asarray(g_idx).astype(np.int64)
        assert g.shape == (k,)
        return g
    return np.arange(k, dtype=np.int64) // groupsize


# -------------------------------------------------------------------------- dequant
def dequant_fp16(qweight, qzeros, scales, groupsize: int, g_idx=None) -> np.ndarray:
    """Canonical dequantised weight, fp16 [K, N]:

        W[k, n] = fp16( float32(q[k,n] - (z[g,n] + 1)) * float32(s[g,n]) ),  g = group(k)

    (README.md:93 `w = (w - z - 1) * s`).  q - z - 1 is an integer in [-16, 14] and the
    scale has an 11-bit significand, so the float32 product is exact and the only
    rounding is float32 -> float16 (round to nearest even).
    """
    q = unpack_qweight(qweight).astype(np.int32)
    z = unpack_qzeros(qzeros).astype(np.int32)
    s = np.asarray(scales, dtype=np.float16)
    k, n = q.shape
    g = group_index(k, groupsize, g_idx)
    assert z.shape[1] == n and s.shape[1] == n and z.shape[0] == s.shape[0]
    assert g.min() >= 0 and g.max() < s.shape[0]
    d = (q - (z[g] + 1)).astype(np.float32)
    return (d * s[g].astype(np.float32)).astype(np.float16)


def dequant_triton_order(qweight, qzeros, scales, groupsize: int) -> np.ndarray:
    """The reference kernel's own rounding order, for documentation only:
    zeros = fp16((z+1)*s); b = fp16(fp16(q*s) - zeros)  (quant_linear.py:188,211-212).
    Up to three fp16 roundings; differs in bits from dequant_fp16 for many (q,z,s)."""
    q = unpack_qweight(qweight).astype(np.float32)
    z = unpack_qzeros(qzeros).astype(np.float32)
    s = np.asarray(scales, dtype=np.float16)
    g = group_index(q.shape[0], groupsize)
    s32 = s[g].astype(np.float32)
    zs = ((z[g] + 1.0) * s32).astype(np.float16)
    qs = (q * s32).astype(np.float16)
    return (qs.astype(np.float32) - zs.astype(np.float32)).astype(np.float16)


# --------------------------------------------------------------------------- matmul
def matmul_ref(x, w_fp16, bias=None) -> np.ndarray:
    """y = x @ W with fp16 operands and wide accumulation, float32 [M, N].

    The reference feeds fp16 tiles to tl.dot with a float32 accumulator and rounds
    once on store (quant_linear.py:194-225).  The oracle accumulates in float64 so it
    carries no summation-order noise of its own; the fp16 rounding of the output and
    the separate fp16 bias add (quant_linear.py:280-281) are applied by matmul_fp16.
    """
    x = np.asarray(x, dtype=np.float16)
    k = x.shape[-1]
    x2 = x.reshape(-1, k).astype(np.float64)
    y = x2 @ np.asarray(w_fp16, dtype=np.float16).astype(np.float64)
    y = y.astype(np.float32)
    if bias is not None:
        y = y + np.asarray(bias, dtype=np.float16).astype(np.float32)
    return y.reshape(x.shape[:-1] + (y.shape[-1],))


def matmul_fp16(x, w_fp16, bias=None) -> np.ndarray:
    """matmul_ref rounded the way the reference rounds: accumulator -> fp16, then an
    fp16 add of the bias (quant_linear.py:225,280-281)."""
    y = matmul_ref(x, w_fp16).astype(np.float16)
    if bias is not None:
        y = (y.astype(np.float32) + np.asarray(bias, np.float16).astype(np.float32)).astype(np.float16)
    return y


def quant_matmul_ref(x, qweight, qzeros, scales, groupsize, bias=None, g_idx=None) -> np.ndarray:
    """triton_matmul4 (quant_linear.py:228-283) as dequantise-then-matmul, float32."""
    return matmul_ref(x, dequant_fp16(qweight, qzeros, scales, groupsize, g_idx), bias)


# ------------------------------------------------------------------------------ MLP
def silu(x: np.ndarray) -> np.ndarray:
    """x * sigmoid(x) (fused_mlp.py:236-238), evaluated in float64."""
    x = np.asarray(x, dtype=np.float64)
    return x / (1.0 + np.exp(-x))


def silu_mul_ref(gate_acc, up_acc) -> np.ndarray:
    """silu(gate) * up on the wide accumulators, float32 (fused_mlp.py:222-225)."""
    return (silu(gate_acc) * np.asarray(up_acc, dtype=np.float64)).astype(np.float32)


def mlp_gateup_ref(x, gate, up, groupsize) -> np.ndarray:
    """triton_llama_mlp_4 (fused_mlp.py:241-302): float32 [.., I] before the fp16 store.
    `gate` and `up` are (qweight, qzeros, scales[, g_idx]) tuples."""
    g = quant_matmul_ref(x, gate[0], gate[1], gate[2], groupsize, g_idx=gate[3] if len(gate) > 3 else None)
    u = quant_matmul_ref(x, up[0], up[1], up[2], groupsize, g_idx=up[3] if len(up) > 3 else None)
    return silu_mul_ref(g, u)


def mlp_ref(x, gate, up, down, groupsize) -> np.ndarray:
    """QuantLlamaMLP.forward (fused_mlp.py:78-79): the fp16-stored intermediate goes
    through down_proj, an ordinary QuantLinear."""
    h = mlp_gateup_ref(x, gate, up, groupsize).astype(np.float16)
    return quant_matmul_ref(h, down[0], down[1], down[2], groupsize, g_idx=down[3] if len(down) > 3 else None)


# --------------------------------------------------------------------------- rotary
def rotary_tables(max_pos: int, head_dim: int = 128, base: float = 10000.0, inv_freq=None):
    """cos, sin float32 [max_pos, head_dim/2].  inv_freq (float32 [head_dim/2]) replaces the computed frequencies
    (the transformers pin passes the library's own, which its float32 pow leaves up to one ulp away).

    inv_freq[i] = float32(base^(-2i/D)), theta[p, i] = float32(p) * inv_freq[i] (a
    float32 product), cos/sin evaluated on that float32 angle and rounded to float32.  (Third-party: transformers'
    LlamaRotaryEmbedding, called at fused_attention.py:101; the table for column
    j >= D/2 repeats column j - D/2.)
    """
    half = head_dim // 2
    # inv_freq is the float32 nearest to the real number base^(-2i/D) (evaluated in
    # float64, rounded once); a float32 pow differs from it by at most one ulp.
    expo = np.arange(0, head_dim, 2, dtype=np.float64) / float(head_dim)
    if inv_freq is None:
        inv_freq = (1.0 / np.power(float(base), expo)).astype(np.float32)
    inv_freq = np.asarray(inv_freq, dtype=np.float32)
    pos = np.arange(max_pos, dtype=np.float32)
    theta = (pos[:, None] * inv_freq[None, :]).astype(np.float32)
    # evaluate the trig functions in float64 on the float32 angle, then round
    cos = np.cos(theta.astype(np.float64)).astype(np.float32)
    sin = np.sin(theta.astype(np.float64)).astype(np.float32)
    assert cos.shape == (max_pos, half)
    return cos, sin


def apply_rotary(x, cos_p, sin_p) -> np.ndarray:
    """Rotate the last axis (size D) by per-row angles; cos_p/sin_p are [..., D/2].

    out[d]      = x[d] * cos[d]      - x[d + D/2] * sin[d]      (d <  D/2)
    out[d+D/2]  = x[d+D/2] * cos[d]  + x[d] * sin[d]
    i.e. q*cos + rotate_half(q)*sin with rotate_half(x) = cat(-x2, x1)
    (apply_rotary_pos_emb as called at fused_attention.py:102).  float64 arithmetic.
    """
    x = np.asarray(x, dtype=np.float64)
    half = x.shape[-1] // 2
    c = np.asarray(cos_p, dtype=np.float64)
    s = np.asarray(sin_p, dtype=np.float64)
    x1, x2 = x[..., :half], x[..., half:]
    return np.concatenate([x1 * c - x2 * s, x2 * c + x1 * s], axis=-1)


def apply_rotary_fp16_order(x_fp16, cos_p, sin_p) -> np.ndarray:
    """The reference-era rounding order: cos/sin cast to fp16, products and the sum
    each rounded to fp16.  Used only to show how far the fp16 order is from the exact
    closed form (a few fp16 ulps)."""
    x = np.asarray(x_fp16, dtype=np.float16)
    half = x.shape[-1] // 2
    c = np.concatenate([cos_p, cos_p], axis=-1).astype(np.float16).astype(np.float32)
    s = np.concatenate([sin_p, sin_p], axis=-1).astype(np.float16).astype(np.float32)
    rot = np.concatenate([-x[..., half:], x[..., :half]], axis=-1).astype(np.float32)
    a = (x.astype(np.float32) * c).astype(np.float16).astype(np.float32)
    b = (rot * s).astype(np.float16).astype(np.float32)
    return (a + b).astype(np.float16)


def qkv_rotary_ref(x, qweight, qzeros, scales, groupsize, position_ids, num_heads, head_dim=128,
                   base=10000.0, g_idx=None, max_pos=None):
    """Fused QKV projection + rotary (fused_attention.py:91-102).

    x: fp16 [B, S, hidden]; packed weights have N = 3*hidden in the order q, k, v
    (fused_attention.py:22-24).  position_ids: int [B, S].
    Returns q, k, v float32 [B, H, S, D]; q and k rotated, v untouched.
    """
    x = np.asarray(x, dtype=np.float16)
    b, s, hidden = x.shape
    assert hidden == num_heads * head_dim
    qkv = quant_matmul_ref(x, qweight, qzeros, scales, groupsize, g_idx=g_idx)  # [B,S,3*hidden]
    assert qkv.shape[-1] == 3 * hidden
    pos = np.asarray(position_ids).reshape(b, s)
    if max_pos is None:
        max_pos = int(pos.max()) + 1
    cos, sin = rotary_tables(max_pos, head_dim, base)
    outs = []
    for i in range(3):
        t = qkv[..., i * hidden:(i + 1) * hidden].reshape(b, s, num_heads, head_dim).transpose(0, 2, 1, 3)
        if i < 2:
            c = cos[pos][:, None, :, :]  # [B,1,S,D/2]
            sn = sin[pos][:, None, :, :]
            t = apply_rotary(t, c, sn)
        outs.append(np.ascontiguousarray(t, dtype=np.float32))
    return tuple(outs)


# ------------------------------------------------------------------- synthetic data
def make_layer(k: int, n: int, groupsize: int, seed: int, act_order: bool = False, bias: bool = False):
    """Seeded synthetic QuantLinear tensors: uniform nibbles, scales uniform in
    [0.002, 0.02] (fp16), optional act-order g_idx = (arange(K)//g)[randperm(K)].
    Returns dict(qweight, qzeros, scales, g_idx|None, bias|None, groupsize)."""
    rng = np.random.default_rng(seed)
    gs = k if groupsize == -1 else groupsize
    g = -(-k // gs)
    qweight = rng.integers(-2**31, 2**31, size=(k // 8, n), dtype=np.int64).astype(np.int32)
    qzeros = rng.integers(-2**31, 2**31, size=(g, n // 8), dtype=np.int64).astype(np.int32)
    scales = (0.002 + 0.018 * rng.random((g, n))).astype(np.float16)
    out = dict(qweight=qweight, qzeros=qzeros, scales=scales, g_idx=None, bias=None, groupsize=groupsize)
    if act_order:
        out["g_idx"] = (np.arange(k) // gs)[rng.permutation(k)].astype(np.int32)
    if bias:
        out["bias"] = rng.standard_normal(n).astype(np.float16)
    return out


def make_x(m: int, k: int, seed: int) -> np.ndarray:
    return np.random.default_rng(seed).standard_normal((m, k)).astype(np.float16)


def within_tolerance(y, y_ref, rtol=1e-2, atol=2e-3):
    """|y - y_ref| <= atol + rtol*|y_ref| elementwise; returns (ok, max_abs, worst_excess)."""
    y = np.asarray(y, dtype=np.float64)
    r = np.asarray(y_ref, dtype=np.float64)
    err = np.abs(y - r)
    lim = atol + rtol * np.abs(r)
    return bool((err <= lim).all()), float(err.max(initial=0.0)), float((err - lim).max(initial=-np.inf))


# ------------------------------------------------------------------ decoder-side operators
def rmsnorm_ref(x: np.ndarray, weight: np.ndarray, eps: float) -> np.ndarray:
    """LLaMA RMSNorm with the module's rounding order: statistics and normalisation in wide
    precision, ONE rounding to fp16, then an fp16 multiply by the weight.  The reference
    runs transformers' LlamaRMSNorm between its fused blocks (the model it patches,
    src/gptq_triton/__init__.py:32-47).  Pinned by: constant rows (y = weight * sign), scale
    invariance for eps = 0, unit-norm rows."""
    xf = np.asarray(x, dtype=np.float64)
    n = (xf / np.sqrt((xf * xf).mean(-1, keepdims=True) + eps)).astype(np.float16)
    return (np.asarray(weight, dtype=np.float16) * n).astype(np.float16)


def decode_attention_ref(q: np.ndarray, k_cache: np.ndarray, v_cache: np.ndarray, positions) -> np.ndarray:
    """One query token per sequence over a KV cache, in float64: for (b, h)
    softmax(q . K[:p+1]^T / sqrt(D)) . V[:p+1] with p = positions[b]; returns [B, 1, H*D]
    (src/gptq_triton/fused_attention.py:118-148 for q_len == 1: scores, fp32 softmax,
    weighted sum, transpose + reshape).  Pinned by: p = 0 gives V[0]; equal keys give the
    mean of V; one key far ahead gives its V row."""
    q = np.asarray(q, dtype=np.float64)
    bsz, heads, _, hd = q.shape
    out = np.zeros((bsz, 1, heads * hd))
    for b in range(bsz):
        p = int(np.asarray(positions).reshape(-1)[b])
        for h in range(heads):
            k = np.asarray(k_cache[b, h, :p + 1], dtype=np.float64)
            v = np.asarray(v_cache[b, h, :p + 1], dtype=np.float64)
            s = k @ q[b, h, 0] / np.sqrt(hd)
            w = np.exp(s - s.max())
            out[b, 0, h * hd:(h + 1) * hd] = (w / w.sum()) @ v
    return out


def prefill_attention_ref(q: np.ndarray, k_cache: np.ndarray, v_cache: np.ndarray, past: int = 0) -> np.ndarray:
    """Causal attention of S query tokens behind `past` cached ones, in float64: query i of (b, h) attends to cache
    rows 0 .. past + i; returns [B, S, H*D] (src/gptq_triton/fused_attention.py:117-141 with the causal mask of
    modeling_llama: scores, mask, fp32 softmax, weighted sum, transpose + reshape).  Pinned by: every query row
    equals decode_attention_ref at position past + i, and torch's scaled_dot_product_attention(is_causal=True) on
    the CPU (tests/test_oracle.py)."""
    q = np.asarray(q, dtype=np.float64)
    bsz, heads, s_len, hd = q.shape
    out = np.zeros((bsz, s_len, heads * hd))
    for b in range(bsz):
        for h in range(heads):
            k = np.asarray(k_cache[b, h, :past + s_len], dtype=np.float64)
            v = np.asarray(v_cache[b, h, :past + s_len], dtype=np.float64)
            sc = q[b, h] @ k.T / np.sqrt(hd)                                       # [S, past + S]
            sc = np.where(np.arange(past + s_len)[None, :] <= past + np.arange(s_len)[:, None], sc, -np.inf)
            w = np.exp(sc - sc.max(axis=1, keepdims=True))
            out[b, :, h * hd:(h + 1) * hd] = (w / w.sum(axis=1, keepdims=True)) @ v
    return out


# ---- streaming order of the packed words (the build's own load-time re-layout; no reference counterpart) ----------
# Pinned by: stream_order_loops (the definition, word by word) == stream_order (index arithmetic) on small shapes;
# unstream(stream_order(q)) == q; and the library's dequantisation FROM the streaming order must reproduce
# dequant_fp16 bit for bit (tests/test_gpu_stream.py), which fails for any wrong index.
def stream_order_loops(qweight: np.ndarray) -> np.ndarray:
    """Definition, word by word: per strip of 16 columns and unit of 128 rows (16 packed rows) one block of 256 words;
    lane l = 16 * r + c owns words 4 * l + j, j = 0..3: packed row unit * 16 + 4 * r + j, column strip * 16 + c."""
    rows, n = qweight.shape
    nb = rows // 16
    out = np.empty(rows * n, dtype=qweight.dtype)
    o = 0
    for strip in range(n // 16):
        for unit in range(nb):
            for r in range(4):
                for c in range(16):
                    for j in range(4):
                        out[o] = qweight[unit * 16 + 4 * r + j, strip * 16 + c]
                        o += 1
    return out.reshape(rows, n)


def stream_order(qweight: np.ndarray, qzeros=None, scales=None):
    """(sweight, smeta): the same permutation by index arithmetic, and the {scale, zero} words
    smeta[(strip * G + g) * 16 + c] = fp16 bits of scales[g, 16 * strip + c] | stored zero << 16."""
    rows, n = qweight.shape
    nb = rows // 16
    o = np.arange(rows * n, dtype=np.int64)
    j, lane, blk = o & 3, (o >> 2) & 63, o >> 8
    strip, unit = blk // nb, blk % nb
    sw = qweight.reshape(-1)[(unit * 16 + 4 * (lane >> 4) + j) * n + strip * 16 + (lane & 15)].reshape(rows, n)
    if scales is None:
        return sw, None
    g = scales.shape[0]
    word = scales.view(np.uint16).astype(np.uint32) | (unpack_qzeros(qzeros).astype(np.uint32) << 16)   # [G, N]
    meta = word.reshape(g, n // 16, 16).transpose(1, 0, 2).reshape(-1).view(np.int32)
    return sw, meta


def unstream(sweight: np.ndarray) -> np.ndarray:
    """The inverse permutation."""
    rows, n = sweight.shape
    nb = rows // 16
    o = np.arange(rows * n, dtype=np.int64)
    j, lane, blk = o & 3, (o >> 2) & 63, o >> 8
    strip, unit = blk // nb, blk % nb
    out = np.empty(rows * n, dtype=sweight.dtype)
    out[(unit * 16 + 4 * (lane >> 4) + j) * n + strip * 16 + (lane & 15)] = sweight.reshape(-1)
    return out.reshape(rows, n)
