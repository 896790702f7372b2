"""GPU parity of the in-place re-rotation of cached K rows against the CPU checker (bit-exact: 16-bit rows and u8
codes / headers), through the C-ABI, plus the eviction -> rotation -> attention flow."""
import numpy as np
import pytest

import harness as H
from oracle import oracle as O

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def dev():
    import torch
    assert torch.cuda.is_available(), "these tests need the MI355X"
    return torch.device("cuda:0")


def _random_cache(rng, nb, Hkv, bs, D, kd):
    x = rng.standard_normal((nb * Hkv * bs, D)).astype(np.float32)
    x[rng.random(x.shape) < 0.01] = 8.0
    if kd == "u8":
        rows = np.stack([O.quantize_row_u8(r) for r in x])
        return rows.reshape(nb, Hkv, bs, D + 8)
    return O.to_bits(x, H.DT[kd]).view(np.uint8).reshape(nb, Hkv, bs, 2 * D)


@pytest.mark.parametrize("kd,D,per_token", [("u8", 128, False), ("u8", 64, True), ("f16", 128, False), ("bf16", 64, False),
                                            ("f16", 64, True), ("bf16", 128, True), ("u8", 256, True), ("bf16", 256, False),
                                            ("u8", 96, False), ("f16", 96, True), ("u8", 192, True), ("bf16", 512, False),
                                            ("u8", 80, False)])
def test_rotate_cache_bit_exact(pkg, dev, kd, D, per_token):
    import torch
    print(f"case rotate {kd} D={D} per_token={per_token}", flush=True)
    rng = np.random.default_rng(21)
    nb, Hkv, bs = 40, 3, 32
    cache = _random_cache(rng, nb, Hkv, bs, D, kd)
    lut = pkg.rotation_trig_lut(bs, 64, D, 10000.0)
    blocks = rng.choice(nb, size=17, replace=False).astype(np.int32)
    deltas = rng.integers(1, 64, size=(17, bs if per_token else 1)).astype(np.int32)
    ref = cache.copy()
    O.rotate_cache(ref, H.DT[kd], blocks, deltas, lut)
    qd = "f16" if kd == "u8" else kd
    op = pkg.PagedAttention(Hkv * 2, Hkv, D, bs, qd, kd, device=0, stream=torch.cuda.current_stream(dev))
    op.set_rotation_trig_lut(lut)
    kc = torch.from_numpy(cache).to(dev)
    op.rotate_cache(kc, blocks, deltas)
    op.synchronize()
    got = kc.cpu().numpy()
    assert np.array_equal(got, ref)
    untouched = np.setdiff1d(np.arange(nb), blocks)
    assert np.array_equal(got[untouched], cache[untouched])
    # nothing to rotate is a no-op
    op.rotate_cache(kc, np.zeros(0, np.int32), np.zeros((0, 1), np.int32))
    op.synchronize()
    assert np.array_equal(kc.cpu().numpy(), ref)


@pytest.mark.parametrize("kd,D", [("u8", 128), ("bf16", 128), ("f16", 64), ("u8", 64)])
def test_rotate_cache_row_count_not_a_multiple_of_a_workgroup(pkg, dev, kd, D):
    """16-token blocks, one kv head, three blocks: 48 rows, so the kernel's last workgroup is half empty."""
    import torch
    print(f"case rotate ragged {kd} D={D}", flush=True)
    rng = np.random.default_rng(22)
    nb, Hkv, bs = 9, 1, 16
    cache = _random_cache(rng, nb, Hkv, bs, D, kd)
    lut = pkg.rotation_trig_lut(bs, 32, D, 10000.0)
    blocks = np.array([7, 0, 4], np.int32)
    deltas = rng.integers(1, 32, size=(3, bs)).astype(np.int32)
    ref = cache.copy()
    O.rotate_cache(ref, H.DT[kd], blocks, deltas, lut)
    qd = "f16" if kd == "u8" else kd
    op = pkg.PagedAttention(4, Hkv, D, bs, qd, kd, device=0, stream=torch.cuda.current_stream(dev))
    op.set_rotation_trig_lut(lut)
    kc = torch.from_numpy(cache).to(dev)
    op.rotate_cache(kc, blocks, deltas)
    op.synchronize()
    assert np.array_equal(kc.cpu().numpy(), ref)


def test_rotate_cache_rejects_bad_arguments(pkg, dev):
    import torch
    op = pkg.PagedAttention(8, 2, 128, 32, "f16", "u8", device=0, stream=torch.cuda.current_stream(dev))
    kc = torch.zeros((4, 2, 32, 136), dtype=torch.uint8, device=dev)
    with pytest.raises(pkg.PaError) as e:  # no table yet
        op.rotate_cache(kc, [1], [[1]])
    assert e.value.status == -10
    op.set_rotation_trig_lut(pkg.rotation_trig_lut(32, 8, 128))
    with pytest.raises(pkg.PaError) as e:  # block outside the cache
        op.rotate_cache(kc, [4], [[1]])
    assert e.value.status == -6
    with pytest.raises(pkg.PaError) as e:  # delta beyond the table
        op.rotate_cache(kc, [1], [[8]])
    assert e.value.status == -6
    with pytest.raises(pkg.PaError) as e:  # neither per block nor per token
        op.rotate_cache(kc, [1, 2], [[1, 1, 1], [1, 1, 1]])
    assert e.value.status == -4
    assert not kc.any()


def test_eviction_then_rotation_keeps_relative_positions(pkg, dev):
    """K rows stored with RoPE at their original positions; blocks 2 and 3 of 8 are evicted, the blocks behind them
    re-rotated: attention of a RoPE'd query then equals attention over a cache that was built at the compacted
    positions in the first place (the relative-position property the rotation exists for)."""
    import torch
    rng = np.random.default_rng(31)
    Hq, Hkv, D, bs, theta = 4, 2, 64, 32, 10000.0
    n_blocks, evicted = 8, [2, 3]
    kept = [b for b in range(n_blocks) if b not in evicted]
    T = n_blocks * bs

    def rope(x, pos):
        ang = pos[:, None] * theta ** (-2.0 * np.arange(D // 2) / D)[None, :]
        a, b = x[..., :D // 2], x[..., D // 2:]
        return np.concatenate([a * np.cos(ang) - b * np.sin(ang), b * np.cos(ang) + a * np.sin(ang)], axis=-1)

    k_raw = rng.standard_normal((T, Hkv, D))
    v_raw = rng.standard_normal((T, Hkv, D))
    pos = np.arange(T, dtype=np.float64)
    k_orig = np.stack([rope(k_raw[:, h], pos) for h in range(Hkv)], axis=1)          # positions as first written
    keep_tok = np.concatenate([np.arange(b * bs, (b + 1) * bs) for b in kept])
    new_pos = np.arange(len(keep_tok), dtype=np.float64)
    k_compact = np.stack([rope(k_raw[keep_tok][:, h], new_pos) for h in range(Hkv)], axis=1)  # built compacted

    def to_cache(k, v):  # [tokens, Hkv, D] -> f16 cache blocks in order
        nb = k.shape[0] // bs
        f = lambda x: O.to_bits(x.reshape(nb, bs, Hkv, D).transpose(0, 2, 1, 3).reshape(-1, D).astype(np.float32),
                                O.DT_F16).view(np.uint8).reshape(nb, Hkv, bs, 2 * D)
        return f(k), f(v)

    kc_orig, vc_orig = to_cache(k_orig, v_raw)
    kc_ref, vc_ref = to_cache(k_compact, v_raw[keep_tok])
    calc = pkg.CacheRotationCalculator(bs, 16, D, theta)
    rot = calc.get_rotation_data(set(evicted), n_blocks)
    assert [r["logical_block_idx"] for r in rot] == [2, 3, 4, 5] and all(r["rotation_delta"] == 2 * bs for r in rot)
    # physical ids = original block numbers; the table after eviction lists the kept blocks
    table = np.array(kept, np.int32)
    op = pkg.PagedAttention(Hq, Hkv, D, bs, "f16", "f16", device=0, stream=torch.cuda.current_stream(dev))
    op.set_rotation_trig_lut(pkg.rotation_trig_lut(bs, 16, D, theta))
    kc = torch.from_numpy(kc_orig).to(dev)
    vc = torch.from_numpy(vc_orig).to(dev)
    op.rotate_cache(kc, table[[r["logical_block_idx"] for r in rot]],
                    np.array([[r["rotation_delta"] // bs] for r in rot], np.int32))
    kv_len = len(keep_tok)
    q = rope(rng.standard_normal((1, Hq, D))[0][None].repeat(1, 0)[0], np.full(Hq, float(kv_len)))  # one token, RoPE at kv_len
    qh = torch.from_numpy(O.to_bits(q.reshape(1, Hq * D).astype(np.float32), O.DT_F16).view(np.int16)).to(dev).view(torch.float16)
    knew = torch.zeros((1, Hkv * D), dtype=torch.float16, device=dev)
    outs = []
    for cache_k, cache_v, tab, nblk in ((kc, vc, table, n_blocks), (torch.from_numpy(kc_ref).to(dev), torch.from_numpy(vc_ref).to(dev),
                                                                     np.arange(len(kept), dtype=np.int32), len(kept))):
        out = torch.zeros((1, Hq * D), dtype=torch.float16, device=dev)
        op.step_begin(np.array([kv_len - 1], np.int32), np.array([0, 1], np.int32), np.array([0, len(tab)], np.int32), kv_len)
        op.set_block_indices(tab, nblk)
        op.attention(qh, cache_k, cache_v, out, None)
        op.synchronize()
        outs.append(out.float().cpu().numpy())
    # the last position (kv_len - 1) is attended in both; two f16 roundings of K on the rotated side
    np.testing.assert_allclose(outs[0], outs[1], rtol=0, atol=4e-3)
