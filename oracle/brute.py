"""Pure-Python brute force used to pin oracle/gptq_oracle.py on tiny inputs.
TEST INFRASTRUCTURE ONLY (same rule as the rest of oracle/).

Nothing here is vectorised and nothing shares code with gptq_oracle: bits are pulled
out one at a time and the dequantised value is computed with exact rationals, then
rounded once to fp16.  A shifted nibble index, a swapped K/N axis, a missing "+1" on
the zero point or a double rounding all show up as a mismatch.
"""
from __future__ import annotations

from fractions import Fraction

import numpy as np


def _bits_of(word: int):
    """32 bits of a signed int32, LSB first."""
    u = word & 0xFFFFFFFF
    return [(u >> i) & 1 for i in range(32)]


def nibble(word: int, t: int) -> int:
    """Field t (0..7, LSB first) of a signed 32-bit container, bit by bit."""
    b = _bits_of(int(word))
    return b[4 * t] | (b[4 * t + 1] << 1) | (b[4 * t + 2] << 2) | (b[4 * t + 3] << 3)


def unpack_qweight_loops(qweight):
    """Row k = 8r + t of column n sits in field t of qweight[r][n]
    (quantize.py:262-271, quant_linear.py:171,177,211)."""
    rows, n = len(qweight), len(qweight[0])
    out = [[0] * n for _ in range(rows * 8)]
    for r in range(rows):
        for c in range(n):
            for t in range(8):
                out[8 * r + t][c] = nibble(qweight[r][c], t)
    return out


def unpack_qzeros_loops(qzeros):
    """Column n = 8c + t of group g sits in field t of qzeros[g][c]
    (quantize.py:276-289, quant_linear.py:178,187)."""
    g, c = len(qzeros), len(qzeros[0])
    out = [[0] * (c * 8) for _ in range(g)]
    for i in range(g):
        for j in range(c):
            for t in range(8):
                out[i][8 * j + t] = nibble(qzeros[i][j], t)
    return out


def fp16_round(fr: Fraction) -> np.float16:
    """Round an exact rational once to fp16 (nearest even).  A Fraction converts to a
    Python float with a single correct rounding; values here are products of a
    5-bit integer and an fp16, so they are exactly representable in float64 and the
    float64 -> float16 conversion is the only rounding."""
    return np.float16(float(fr))


def dequant_loops(qweight, qzeros, scales, groupsize, g_idx=None):
    """W[k][n] = fp16((q - (z + 1)) * s) with exact rational arithmetic (README.md:93)."""
    q = unpack_qweight_loops(qweight)
    z = unpack_qzeros_loops(qzeros)
    k, n = len(q), len(q[0])
    if groupsize == -1:
        groupsize = k
    out = np.empty((k, n), dtype=np.float16)
    for i in range(k):
        g = int(g_idx[i]) if g_idx is not None else i // groupsize
        for j in range(n):
            s = Fraction(float(scales[g][j]))
            out[i, j] = fp16_round((q[i][j] - (z[g][j] + 1)) * s)
    return out


def matmul_loops(x, w):
    """y[m][n] = sum_k x[m][k] * w[k][n] in exact rationals, returned as float64."""
    m, k, n = len(x), len(w), len(w[0])
    out = np.empty((m, n), dtype=np.float64)
    for i in range(m):
        for j in range(n):
            acc = Fraction(0)
            for t in range(k):
                acc += Fraction(float(x[i][t])) * Fraction(float(w[t][j]))
            out[i, j] = float(acc)
    return out
