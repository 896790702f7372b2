"""Pins the CPU checker's KV-append / quantisation / attention restatement with what the mathematics fixes:
exact-rational quantisation on small rows, brute-force gathers, float64 textbook attention and torch SDPA."""
import numpy as np
import pytest

import ref_math as R
from oracle import oracle as O


def _mk_case(rng, B, Hq, Hkv, D, bs, cache_dtype, q_dtype, past_rng, new_rng, pool_factor=2):
    past = rng.integers(past_rng[0], past_rng[1] + 1, size=B).astype(np.int32)
    new = rng.integers(new_rng[0], new_rng[1] + 1, size=B).astype(np.int32)
    sb = np.concatenate([[0], np.cumsum(new)]).astype(np.int32)
    nblk = (past + new + bs - 1) // bs
    bib = np.concatenate([[0], np.cumsum(nblk)]).astype(np.int32)
    pool = int(pool_factor * bib[-1]) + 1
    table = rng.permutation(pool)[:bib[-1]].astype(np.int32)
    T = int(sb[-1])
    rb = O.row_bytes(D, cache_dtype)
    kc = np.zeros((pool, Hkv, bs, rb), np.uint8)
    vc = np.zeros((pool, Hkv, bs, rb), np.uint8)
    src_dtype = q_dtype
    # fill the past through the checker's own append (prefill of `past` tokens per sequence)
    if past.sum() > 0:
        psb = np.concatenate([[0], np.cumsum(past)]).astype(np.int32)
        kp = O.to_bits(rng.standard_normal((int(psb[-1]), Hkv * D)).astype(np.float32), src_dtype)
        vp = O.to_bits(rng.standard_normal((int(psb[-1]), Hkv * D)).astype(np.float32), src_dtype)
        O.kv_append(kp, vp, src_dtype, kc, vc, cache_dtype, np.zeros(B, np.int32), psb, table, bib, Hkv, D, bs)
    q = O.to_bits(rng.standard_normal((T, Hq * D)).astype(np.float32), q_dtype)
    k = O.to_bits(rng.standard_normal((T, Hkv * D)).astype(np.float32), src_dtype)
    v = O.to_bits(rng.standard_normal((T, Hkv * D)).astype(np.float32), src_dtype)
    return dict(past=past, sb=sb, bib=bib, table=table, kc=kc, vc=vc, q=q, k=k, v=v, pool=pool)


def _rows_f32(cache, table, kv_len, h, bs, cache_dtype):
    rows = R.gather_rows(cache, table, kv_len, h, bs)
    if cache_dtype == O.DT_U8:
        return R.dequant_rows_u8(rows)
    return O.from_bits(rows.reshape(kv_len, -1).view(np.uint16), cache_dtype)


# ------------------------------------------------------------------------------------------- 16-bit conversions
def test_half_conversions_match_numpy():
    bits = np.arange(0, 1 << 16, dtype=np.uint16)
    ref = bits.view(np.float16).astype(np.float32)
    L = O.lib()
    for b in list(range(0, 1 << 16, 97)) + [0, 1, 0x3ff, 0x400, 0x7bff, 0x7c00, 0x8000, 0x8001, 0xfbff, 0xfc00]:
        got = L.orc_half_to_float(int(b))
        if np.isnan(ref[b]):
            assert np.isnan(got)
        else:
            assert got == ref[b]
    rng = np.random.default_rng(5)
    vals = np.concatenate([rng.standard_normal(500) * 10.0 ** rng.integers(-9, 6, 500),
                           [0.0, 65504.0, 65519.9, 65520.0, 1e-8, 5.96e-8, 2.98e-8, 2.9802322e-8, 6.1e-5, 1e6]])
    for v in vals.astype(np.float32):
        assert L.orc_float_to_half(float(v)) == int(np.float32(v).astype(np.float16).view(np.uint16)), v
    for v in vals.astype(np.float32):
        b = L.orc_float_to_bf16(float(v))
        assert b == int(O.f32_to_bf16_bits(np.array([v]))[0])
        assert L.orc_bf16_to_float(b) == O.bf16_bits_to_f32(np.array([b], np.uint16))[0]


# ------------------------------------------------------------------------------------------- u8 rows
@pytest.mark.parametrize("seed", range(6))
def test_quantize_row_matches_exact_rational(seed):
    rng = np.random.default_rng(100 + seed)
    D = [8, 16, 64, 128, 24, 128][seed]
    x = rng.standard_normal(D).astype(np.float16).astype(np.float32)
    if seed == 5:
        x[rng.integers(0, D, 3)] = np.float32([8.0, -8.0, 8.0])
    row = O.quantize_row_u8(x)
    scale, zp, codes = R.quantize_row_exact(x)
    assert row[:4].view(np.float32)[0] == scale
    assert row[4:8].view(np.float32)[0] == zp
    assert list(row[8:]) == codes


def test_quantize_row_ties_round_to_even():
    # min 0, max 255 -> scale 1, zp 0, inverse 1: x + 0 is exact, so halves are exact ties
    x = np.array([0.0, 255.0, 0.5, 1.5, 2.5, 3.5, 126.5, 127.5, 254.5, 100.25, 100.75], np.float32)
    row = O.quantize_row_u8(x)
    assert row[:8].view(np.float32).tolist() == [1.0, 0.0]
    assert list(row[8:]) == [0, 255, 0, 2, 2, 4, 126, 128, 254, 100, 101]


def test_quantize_row_invariants():
    rng = np.random.default_rng(7)
    for _ in range(50):
        D = int(rng.choice([64, 128]))
        x = (rng.standard_normal(D) * rng.uniform(0.01, 30)).astype(np.float16).astype(np.float32)
        row = O.quantize_row_u8(x)
        scale, zp = row[:8].view(np.float32)
        codes = row[8:].astype(np.float32)
        assert codes[np.argmin(x)] == 0 and codes[np.argmax(x)] == 255
        deq = (codes - zp) * scale
        assert np.all(np.abs(deq - x) <= 0.5 * scale * (1 + 1e-3) + 1e-6)
    # a constant row takes scale 1e-4 and code 0 everywhere; the value sits in the zero point
    row = O.quantize_row_u8(np.full(64, 1.25, np.float32))
    scale, zp = row[:8].view(np.float32)
    assert scale == np.float32(0.0001) and zp == np.float32(-1.25) / np.float32(0.0001)
    assert not row[8:].any()
    assert abs((0 - zp) * scale - 1.25) < 1e-6


# ------------------------------------------------------------------------------------------- append = scatter
# ------------------------------------------------------------------------------------------- u4 rows
@pytest.mark.parametrize("seed", range(5))
def test_quantize_row_u4_matches_exact_rational(seed):
    rng = np.random.default_rng(300 + seed)
    D = [8, 16, 80, 128, 256][seed]
    x = rng.standard_normal(D).astype(np.float16).astype(np.float32)
    if seed == 3:
        x[rng.integers(0, D, 3)] = np.float32([8.0, -8.0, 8.0])
    row = O.quantize_row_u4(x)
    assert row.size == D // 2 + 8
    scale, zp, codes = R.quantize_row_exact(x, levels=15)
    assert row[:4].view(np.float32)[0] == scale
    assert row[4:8].view(np.float32)[0] == zp
    got = np.stack([row[8:] >> 4, row[8:] & 15], axis=1).reshape(-1)  # element 2 i in the high nibble of byte i
    assert list(got) == codes


def test_quantize_row_u4_invariants():
    rng = np.random.default_rng(8)
    for D in (8, 64, 96, 128):
        x = (rng.standard_normal(D) * 3).astype(np.float32)
        row = O.quantize_row_u4(x)
        sc, zp = row[:8].view(np.float32)
        codes = np.stack([row[8:] >> 4, row[8:] & 15], axis=1).reshape(-1)
        assert codes.min() == 0 and codes.max() == 15  # the extremes land on the ends of the range
        assert np.argmin(x) in np.flatnonzero(codes == 0) and np.argmax(x) in np.flatnonzero(codes == 15)
        deq = (codes.astype(np.float32) - zp) * sc
        assert np.all(np.abs(deq - x) <= 0.5 * sc * 1.001 + 1e-6)  # half a quantisation step
        assert np.array_equal(R.dequant_rows_u4(row[None])[0], deq)
    const = O.quantize_row_u4(np.full(16, 2.5, np.float32))  # a zero range takes the fixed scale
    assert const[:4].view(np.float32)[0] == np.float32(0.0001)
    # exact ties round to even: min 0, max 15 -> scale 1, zp 0
    x = np.array([0.0, 15.0, 0.5, 1.5, 2.5, 3.5, 13.5, 14.5], np.float32)
    row = O.quantize_row_u4(x)
    assert list(np.stack([row[8:] >> 4, row[8:] & 15], axis=1).reshape(-1)) == [0, 15, 0, 2, 2, 4, 14, 14]


KV_MIXES = [
    # (Dk, Dv, key cache type, value cache type): head sizes and precisions that differ between the two tensors
    (80, 80, "f16", "f16"), (96, 96, "u8", "u8"), (256, 256, "bf16", "bf16"), (128, 64, "u8", "f16"),
    (64, 128, "f16", "u8"), (192, 128, "bf16", "u4"), (128, 128, "u4", "u4"), (72, 40, "u4", "bf16"),
]


@pytest.mark.parametrize("Dk,Dv,kd,vd", KV_MIXES)
def test_attention_with_a_head_size_and_type_per_tensor_matches_float64(Dk, Dv, kd, vd):
    """The per-tensor form of the checker (key rows of Dk elements in one type, value rows of Dv in another) against
    the float64 textbook form over rows dequantised independently here; the append is checked row by row."""
    dts = {"f16": O.DT_F16, "bf16": O.DT_BF16, "u8": O.DT_U8, "u4": O.DT_U4}
    kdt, vdt = dts[kd], dts[vd]
    qdt = O.DT_BF16 if "bf16" in (kd, vd) else O.DT_F16
    rng = np.random.default_rng(Dk * 7 + Dv)
    B, Hq, Hkv, bs = 3, 6, 2, 16
    G = Hq // Hkv
    past = np.array([0, 37, 90], np.int32)
    new = np.array([21, 1, 5], np.int32)
    sb = np.concatenate([[0], np.cumsum(new)]).astype(np.int32)
    nblk = (past + new + bs - 1) // bs
    bib = np.concatenate([[0], np.cumsum(nblk)]).astype(np.int32)
    pool = 2 * int(bib[-1]) + 1
    table = rng.permutation(pool)[:bib[-1]].astype(np.int32)
    kc = np.zeros((pool, Hkv, bs, O.row_bytes(Dk, kdt)), np.uint8)
    vc = np.zeros((pool, Hkv, bs, O.row_bytes(Dv, vdt)), np.uint8)
    tot = past + new
    asb = np.concatenate([[0], np.cumsum(tot)]).astype(np.int32)
    k_all = rng.standard_normal((int(asb[-1]), Hkv, Dk)).astype(np.float32)
    v_all = rng.standard_normal((int(asb[-1]), Hkv, Dv)).astype(np.float32)
    kb, vb = O.to_bits(k_all.reshape(-1, Hkv * Dk), qdt), O.to_bits(v_all.reshape(-1, Hkv * Dv), qdt)
    O.kv_append_kv(kb, vb, qdt, kc, vc, kdt, vdt, np.zeros(B, np.int32), asb, table, bib, Hkv, Dk, Dv, bs)

    def rows(cache, D, dt, b, h):
        r = R.gather_rows(cache, table[bib[b]:bib[b + 1]], int(tot[b]), h, bs)
        if dt == O.DT_U8:
            return R.dequant_rows_u8(r)
        if dt == O.DT_U4:
            return R.dequant_rows_u4(r)
        return O.from_bits(r.reshape(int(tot[b]), -1).view(np.uint16), dt)

    # the append: every row is what its type's recipe makes of the source row
    src_k = O.from_bits(kb, qdt).reshape(-1, Hkv, Dk)
    src_v = O.from_bits(vb, qdt).reshape(-1, Hkv, Dv)
    for b in range(B):
        for h in range(Hkv):
            for cache, D, dt, src in ((kc, Dk, kdt, src_k), (vc, Dv, vdt, src_v)):
                got = R.gather_rows(cache, table[bib[b]:bib[b + 1]], int(tot[b]), h, bs)
                for j in (0, int(tot[b]) - 1):
                    x = src[asb[b] + j, h]
                    if dt == O.DT_U8:
                        assert np.array_equal(got[j], O.quantize_row_u8(x))
                    elif dt == O.DT_U4:
                        assert np.array_equal(got[j], O.quantize_row_u4(x))
                    else:
                        assert np.array_equal(got[j].view(np.uint16), O.to_bits(x[None], dt)[0])
    q = O.to_bits(rng.standard_normal((int(sb[-1]), Hq * Dk)).astype(np.float32), qdt)
    scale = float(1.0 / np.sqrt(Dk))
    W = np.array([3, 1, 2], np.int32)
    out, out16, scores = O.paged_attention_kv(q, qdt, kc, vc, kdt, vdt, past, sb, table, bib, Hq, Hkv, Dk, Dv, bs, scale,
                                              0, W, True, 4)
    assert out.shape == (int(sb[-1]), Hq * Dv)
    qf = O.from_bits(q, qdt).reshape(-1, Hq, Dk)
    so = np.concatenate([[0], np.cumsum(tot)])
    for b in range(B):
        sc_ref = np.zeros(int(tot[b]))
        for h in range(Hkv):
            o, s = R.attention_f64(qf[sb[b]:sb[b + 1], h * G:(h + 1) * G], rows(kc, Dk, kdt, b, h), rows(vc, Dv, vdt, b, h),
                                   int(past[b]), scale, 0, int(W[b]))
            got = out[sb[b]:sb[b + 1]].reshape(-1, Hq, Dv)[:, h * G:(h + 1) * G]
            np.testing.assert_allclose(got, o, rtol=2e-5, atol=2e-5)
            sc_ref += s
        np.testing.assert_allclose(scores[so[b]:so[b + 1]], sc_ref, rtol=2e-5, atol=2e-5)
    # ... with the op's alibi_slopes input: logit += slope[head] * (key position - query position), against the
    # float64 form; with a sliding window on top; zero slopes give the bits of the form without slopes
    slopes = (2.0 ** -(np.arange(Hq) * 8.0 / Hq + 1)).astype(np.float32) * np.where(np.arange(Hq) % 3 == 2, 0.0, 1.0).astype(np.float32)
    for sw in (0, 13):
        out_a, _, scores_a = O.paged_attention_alibi(q, qdt, kc, vc, kdt, vdt, past, sb, table, bib, Hq, Hkv, Dk, Dv, bs,
                                                     scale, slopes, sw, W, True, 4)
        assert np.abs(out_a - out).max() > 1e-3   # (the slopes matter on this data)
        for b in range(B):
            sc_ref = np.zeros(int(tot[b]))
            for h in range(Hkv):
                o, s = R.attention_f64(qf[sb[b]:sb[b + 1], h * G:(h + 1) * G], rows(kc, Dk, kdt, b, h),
                                       rows(vc, Dv, vdt, b, h), int(past[b]), scale, sw, int(W[b]), slopes[h * G:(h + 1) * G])
                got = out_a[sb[b]:sb[b + 1]].reshape(-1, Hq, Dv)[:, h * G:(h + 1) * G]
                np.testing.assert_allclose(got, o, rtol=2e-5, atol=2e-5)
                sc_ref += s
            np.testing.assert_allclose(scores_a[so[b]:so[b + 1]], sc_ref, rtol=2e-5, atol=2e-5)
    out_z, out16_z, scores_z = O.paged_attention_alibi(q, qdt, kc, vc, kdt, vdt, past, sb, table, bib, Hq, Hkv, Dk, Dv, bs,
                                                       scale, np.zeros(Hq, np.float32), 0, W, True, 4)
    assert np.array_equal(out16_z, out16) and np.array_equal(scores_z, scores)
    # ... and equal head sizes and types give the bits of the plain form
    if Dk == Dv and kdt == vdt and kdt != O.DT_U4:
        out2, out16_2, scores2 = O.paged_attention(q, qdt, kc, vc, kdt, past, sb, table, bib, Hq, Hkv, Dk, bs, scale, 0, W,
                                                   True, 4)
        assert np.array_equal(out16, out16_2) and np.array_equal(scores, scores2)


@pytest.mark.parametrize("cache_dtype,src_dtype", [(O.DT_U8, O.DT_F16), (O.DT_F16, O.DT_F16), (O.DT_BF16, O.DT_BF16),
                                                   (O.DT_U8, O.DT_BF16)])
def test_kv_append_is_a_paged_scatter(cache_dtype, src_dtype):
    rng = np.random.default_rng(11)
    B, Hkv, D, bs = 5, 2, 64, 32
    c = _mk_case(rng, B, 4, Hkv, D, bs, cache_dtype, src_dtype, (0, 70), (1, 40))
    kc0, vc0 = c["kc"].copy(), c["vc"].copy()
    O.kv_append(c["k"], c["v"], src_dtype, c["kc"], c["vc"], cache_dtype, c["past"], c["sb"], c["table"], c["bib"],
                Hkv, D, bs)
    touched = np.zeros(c["kc"].shape[:3], bool)
    for b in range(B):
        tab = c["table"][c["bib"][b]:c["bib"][b + 1]]
        for t in range(c["sb"][b + 1] - c["sb"][b]):
            slot = c["past"][b] + t
            for h in range(Hkv):
                for src, cache in ((c["k"], c["kc"]), (c["v"], c["vc"])):
                    x = src[c["sb"][b] + t, h * D:(h + 1) * D]
                    got = cache[tab[slot // bs], h, slot % bs]
                    if cache_dtype == O.DT_U8:
                        exp = O.quantize_row_u8(O.from_bits(x, src_dtype))
                    else:
                        exp = x.view(np.uint8)
                    assert np.array_equal(got, exp)
                touched[tab[slot // bs], h, slot % bs] = True
    # every other slot is untouched
    assert np.array_equal(c["kc"][~touched], kc0[~touched])
    assert np.array_equal(c["vc"][~touched], vc0[~touched])


def test_kv_append_rejects_bad_tables():
    rng = np.random.default_rng(3)
    c = _mk_case(rng, 2, 4, 2, 64, 32, O.DT_F16, O.DT_F16, (10, 20), (1, 1))
    bad = c["table"].copy()
    bad[0] = c["pool"] + 5
    with pytest.raises(RuntimeError):
        O.kv_append(c["k"], c["v"], O.DT_F16, c["kc"], c["vc"], O.DT_F16, c["past"], c["sb"], bad, c["bib"], 2, 64, 32)


# ------------------------------------------------------------------------------------------- attention
CASES = [
    # B, Hq, Hkv, D, bs, cache, q, past range, new range, sliding window, W
    (4, 8, 2, 64, 32, O.DT_F16, O.DT_F16, (1, 150), (1, 1), 0, None),
    (3, 8, 2, 128, 32, O.DT_U8, O.DT_F16, (30, 200), (1, 1), 0, None),
    (3, 14, 2, 128, 32, O.DT_BF16, O.DT_BF16, (0, 100), (1, 48), 0, "mixed"),
    (3, 10, 2, 128, 32, O.DT_U8, O.DT_F16, (100, 300), (1, 1), 64, None),
    (2, 4, 4, 64, 16, O.DT_F16, O.DT_F16, (0, 40), (5, 40), 24, "mixed"),
    (2, 8, 8, 64, 32, O.DT_U8, O.DT_BF16, (0, 0), (1, 33), 0, "zero"),
]


@pytest.mark.parametrize("case", CASES, ids=lambda c: f"B{c[0]}_Hq{c[1]}_Hkv{c[2]}_D{c[3]}_c{c[5]}_sw{c[9]}")
def test_attention_matches_float64_textbook(case):
    B, Hq, Hkv, D, bs, cache_dtype, q_dtype, past_rng, new_rng, sw, wmode = case
    rng = np.random.default_rng(42)
    c = _mk_case(rng, B, Hq, Hkv, D, bs, cache_dtype, q_dtype, past_rng, new_rng)
    O.kv_append(c["k"], c["v"], q_dtype, c["kc"], c["vc"], cache_dtype, c["past"], c["sb"], c["table"], c["bib"],
                Hkv, D, bs)
    new = np.diff(c["sb"])
    if wmode is None:
        saw = None
        W = np.ones(B, np.int64)
    elif wmode == "zero":
        saw = np.zeros(B, np.int32)
        W = saw
    else:
        saw = np.array([rng.integers(0, n + 1) for n in new], np.int32)
        W = saw
    scale = 1.0 / np.sqrt(D)
    out, out16, scores = O.paged_attention(c["q"], q_dtype, c["kc"], c["vc"], cache_dtype, c["past"], c["sb"],
                                           c["table"], c["bib"], Hq, Hkv, D, bs, scale, sw, saw, True, num_threads=4)
    G = Hq // Hkv
    qf = O.from_bits(c["q"], q_dtype).reshape(-1, Hkv, G, D)
    off = 0
    for b in range(B):
        kv_len = int(c["past"][b] + new[b])
        tab = c["table"][c["bib"][b]:c["bib"][b + 1]]
        sc = np.zeros(kv_len)
        for h in range(Hkv):
            Kr = _rows_f32(c["kc"], tab, kv_len, h, bs, cache_dtype)
            Vr = _rows_f32(c["vc"], tab, kv_len, h, bs, cache_dtype)
            o, s = R.attention_f64(qf[c["sb"][b]:c["sb"][b + 1], h], Kr, Vr, int(c["past"][b]), scale, sw, int(W[b]))
            got = out[c["sb"][b]:c["sb"][b + 1]].reshape(-1, Hkv, G, D)[:, h]
            np.testing.assert_allclose(got, o, rtol=2e-5, atol=2e-5)
            sc += s
        np.testing.assert_allclose(scores[off:off + kv_len], sc, rtol=2e-5, atol=2e-5)
        # each softmax row sums to one: total mass = Hq * W rows (rows see at least one position)
        assert abs(scores[off:off + kv_len].sum() - Hq * min(int(W[b]), int(new[b]))) < 1e-3 * Hq
        off += kv_len
    # the 16-bit output is the float output rounded once to the query dtype
    assert np.array_equal(out16, O.to_bits(out, q_dtype))


def test_attention_matches_torch_sdpa():
    torch = pytest.importorskip("torch")
    rng = np.random.default_rng(9)
    B, Hq, Hkv, D, bs = 3, 8, 2, 64, 32
    c = _mk_case(rng, B, Hq, Hkv, D, bs, O.DT_F16, O.DT_F16, (5, 90), (1, 20))
    O.kv_append(c["k"], c["v"], O.DT_F16, c["kc"], c["vc"], O.DT_F16, c["past"], c["sb"], c["table"], c["bib"], Hkv, D, bs)
    scale = 0.11
    out, _, _ = O.paged_attention(c["q"], O.DT_F16, c["kc"], c["vc"], O.DT_F16, c["past"], c["sb"], c["table"],
                                  c["bib"], Hq, Hkv, D, bs, scale, 0, None, False)
    G = Hq // Hkv
    for b in range(B):
        q_len = int(c["sb"][b + 1] - c["sb"][b])
        kv_len = int(c["past"][b]) + q_len
        tab = c["table"][c["bib"][b]:c["bib"][b + 1]]
        K = np.stack([_rows_f32(c["kc"], tab, kv_len, h, bs, O.DT_F16) for h in range(Hkv)])  # [Hkv, kv, D]
        V = np.stack([_rows_f32(c["vc"], tab, kv_len, h, bs, O.DT_F16) for h in range(Hkv)])
        q = O.from_bits(c["q"][c["sb"][b]:c["sb"][b + 1]], O.DT_F16).reshape(q_len, Hq, D).transpose(1, 0, 2)
        Kt = torch.from_numpy(K).repeat_interleave(G, dim=0)
        Vt = torch.from_numpy(V).repeat_interleave(G, dim=0)
        mask = torch.ones(q_len, kv_len, dtype=torch.bool).tril(diagonal=int(c["past"][b]))
        ref = torch.nn.functional.scaled_dot_product_attention(torch.from_numpy(q.copy())[None], Kt[None], Vt[None],
                                                               attn_mask=mask, scale=scale)[0]
        got = out[c["sb"][b]:c["sb"][b + 1]].reshape(q_len, Hq, D).transpose(1, 0, 2)
        np.testing.assert_allclose(got, ref.numpy(), rtol=2e-5, atol=2e-5)


def test_paged_read_is_permutation_invariant():
    # the same logical content under two different physical placements gives identical results
    rng = np.random.default_rng(21)
    B, Hq, Hkv, D, bs = 2, 4, 2, 64, 32
    c = _mk_case(rng, B, Hq, Hkv, D, bs, O.DT_U8, O.DT_F16, (40, 90), (1, 1))
    O.kv_append(c["k"], c["v"], O.DT_F16, c["kc"], c["vc"], O.DT_U8, c["past"], c["sb"], c["table"], c["bib"], Hkv, D, bs)
    a = O.paged_attention(c["q"], O.DT_F16, c["kc"], c["vc"], O.DT_U8, c["past"], c["sb"], c["table"], c["bib"],
                          Hq, Hkv, D, bs, 0.125)
    perm = rng.permutation(c["pool"])
    inv = np.argsort(perm)  # new physical id of old block p is inv[p]
    kc2, vc2 = c["kc"][perm], c["vc"][perm]
    table2 = inv[c["table"]].astype(np.int32)
    b = O.paged_attention(c["q"], O.DT_F16, kc2, vc2, O.DT_U8, c["past"], c["sb"], table2, c["bib"],
                          Hq, Hkv, D, bs, 0.125)
    assert np.array_equal(a[0], b[0]) and np.array_equal(a[2], b[2])


def test_pack_step_and_block_count_normalisation():
    # model_runner.hpp:802-822 closed form
    past, sb, bib, mx = O.pack_step([100, 64, 0], [32, 0, 0], [0, 1, 0], [1, 1, 40], [3, 3, 2], 32)
    assert past.tolist() == [68, 32, 0] and sb.tolist() == [0, 1, 2, 42] and bib.tolist() == [0, 3, 5, 7] and mx == 101
    # cache_orchestrator.hpp:814-850: 1 GiB of 1 MiB blocks = 1024 blocks; explicit count wins over cache_size
    assert O.normalize_num_kv_blocks(0, 1, 32, 1 << 20, 1 << 40) == 1024
    assert O.normalize_num_kv_blocks(77, 1, 32, 1 << 20, 1 << 40) == 77
    assert O.normalize_num_kv_blocks(0, 0, 32, 1 << 20, 1 << 40) == 0
    assert O.normalize_num_kv_blocks(0, 1, 32, 3 << 19, 1 << 40) == (1 << 30) // (3 << 19)
    with pytest.raises(RuntimeError):
        O.normalize_num_kv_blocks(0, 4, 32, 1 << 20, 1 << 30)
