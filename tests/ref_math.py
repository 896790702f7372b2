"""Independent float64 / exact-rational restatements used to pin the CPU checker (never the product)."""
from fractions import Fraction

import numpy as np


def frac_to_f32(fr):
    """Correctly rounded (ties to even) float32 of an exact rational."""
    if fr == 0:
        return np.float32(0.0)
    sign = -1 if fr < 0 else 1
    a = abs(fr)
    e = 0
    # find e with 2^e <= a < 2^(e+1)
    while a >= 2:
        a /= 2
        e += 1
    while a < 1:
        a *= 2
        e -= 1
    e = max(e, -126)  # subnormal range keeps the exponent fixed
    scaled = abs(fr) / Fraction(2) ** (e - 23)
    n = scaled.numerator // scaled.denominator
    rem = scaled - n
    if rem > Fraction(1, 2) or (rem == Fraction(1, 2) and (n & 1)):
        n += 1
    return np.float32(sign * float(Fraction(n) * Fraction(2) ** (e - 23)))


def quantize_row_exact(x, levels=255):
    """u8 (``levels`` 255) or u4 (15) row of ``x`` (float32 values) by exact rational arithmetic: scale, zp, codes."""
    x = [np.float32(v) for v in x]
    mn, mx = min(x), max(x)
    # (mx - mn) is itself rounded to float32 before the division
    diff = frac_to_f32(Fraction(float(mx)) - Fraction(float(mn)))
    scale = frac_to_f32(Fraction(float(diff)) / levels)
    if scale == 0:
        scale = np.float32(0.0001)
    zp = frac_to_f32(-Fraction(float(mn)) / Fraction(float(scale)))
    inv = frac_to_f32(Fraction(1) / Fraction(float(scale)))
    codes = []
    for v in x:
        t = frac_to_f32(Fraction(float(v)) * Fraction(float(inv)) + Fraction(float(zp)))  # fused multiply-add
        t = float(t)
        r = np.floor(t)
        d = t - r
        if d > 0.5 or (d == 0.5 and int(r) % 2 == 1):
            r += 1
        codes.append(int(min(max(r, 0), levels)))
    return scale, zp, codes


def gather_rows(cache, table, kv_len, h, bs):
    """cache [num_blocks, Hkv, bs, ...] -> rows [kv_len, ...] of head h following the block table."""
    return np.stack([cache[table[j // bs], h, j % bs] for j in range(kv_len)])


def dequant_rows_u8(rows):
    """rows uint8 [n, D+8] -> float32 [n, D] as (code - zp) * scale in float32."""
    hdr = rows[:, :8].copy().view(np.float32)
    scale, zp = hdr[:, 0:1], hdr[:, 1:2]
    return (rows[:, 8:].astype(np.float32) - zp) * scale


def dequant_rows_u4(rows):
    """rows uint8 [n, D/2+8] -> float32 [n, D]: element 2 i from the high nibble of byte i, 2 i + 1 from the low one."""
    hdr = rows[:, :8].copy().view(np.float32)
    scale, zp = hdr[:, 0:1], hdr[:, 1:2]
    codes = np.stack([rows[:, 8:] >> 4, rows[:, 8:] & 15], axis=2).reshape(rows.shape[0], -1)
    return (codes.astype(np.float32) - zp) * scale


def attention_f64(q, K, V, past, scale, sliding_window, W, slopes=None):
    """Textbook attention in float64 for one sequence and one kv head.

    q [q_len, G, D], K [kv_len, D], V [kv_len, Dv] -> out [q_len, G, Dv], scores [kv_len] (sum over G heads and
    last W rows).  slopes [G]: ALiBi, logit += slope * (key position - query position).
    """
    q = q.astype(np.float64)
    K = K.astype(np.float64)
    V = V.astype(np.float64)
    q_len, G, D = q.shape
    kv_len = K.shape[0]
    out = np.zeros((q_len, G, V.shape[1]))
    scores = np.zeros(kv_len)
    for i in range(q_len):
        last = past + i
        first = max(0, last + 1 - sliding_window) if sliding_window > 0 else 0
        s = (q[i] @ K[first:last + 1].T) * scale  # [G, n]
        if slopes is not None:
            s = s + np.asarray(slopes, np.float64)[:, None] * (np.arange(first, last + 1) - last)[None, :]
        s -= s.max(axis=1, keepdims=True)
        p = np.exp(s)
        p /= p.sum(axis=1, keepdims=True)
        out[i] = p @ V[first:last + 1]
        if i >= q_len - W:
            scores[first:last + 1] += p.sum(axis=0)
    return out, scores
