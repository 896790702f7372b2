"""Block diversity of the evictable area on the GPU (matrix cores; the vector unit for shapes the matrix-core kernels
are not built for) against the CPU checker on the same paged key caches.  Tolerance 2e-3 relative / 1e-3 absolute, plus the checker's own slack for similarities that sit within
2e-5 of their row's mean (dropping entries below the mean is a step function: a value computed in f32 may fall on
the other side of it)."""
import numpy as np
import pytest

import rkv_diversity_cases as RC
from oracle import oracle as O

pytestmark = pytest.mark.gpu
RTOL, ATOL, MARGIN = 2e-3, 1e-3, 2e-5


def _run(pkg, kv, q, Hq, Hkv, D, lens, start, ev_sizes, seed, keys=None, bs=32):
    import torch
    dev = torch.device("cuda:0")
    rng = np.random.default_rng(seed)
    kc, ids, bib = RC.paged_key_cache(rng, lens, Hkv, D, bs, kv, q, keys=keys)
    B = len(lens)
    op = pkg.PagedAttention(Hq, Hkv, D, bs, q, kv, num_layers=2, device=0, stream=torch.cuda.current_stream(dev))
    # a decode step whose new token is the last of `lens`
    past = (np.asarray(lens) - 1).astype(np.int32)
    op.step_begin(past, np.arange(B + 1, dtype=np.int32), bib)
    op.set_block_indices(ids, kc.shape[0], layer=1)
    op.set_block_indices(ids[::-1].copy(), kc.shape[0], layer=0)  # layer 0 gets another table: must not be used
    kc_d = torch.from_numpy(kc).to(dev)
    total = sum((e // bs) * e for e in ev_sizes)
    out = torch.full((total + 7,), 123.0, device=dev)
    offsets = op.adaptive_rkv_diversity(kc_d, start, ev_sizes, out, layer=1)
    op.synchronize()
    got = out.cpu().numpy()
    assert np.all(got[total:] == 123.0)  # nothing written past the areas
    assert offsets[-1] == total
    results = []
    for b in range(B):
        ev = ev_sizes[b]
        assert offsets[b + 1] - offsets[b] == (ev // bs) * ev
        if ev == 0:
            continue
        ref, slack = O.adaptive_rkv_diversity(kc, RC.DT[kv], Hkv, bs, D, ids[bib[b]:bib[b + 1]], start, ev, margin=MARGIN)
        g = got[offsets[b]:offsets[b + 1]].reshape(ev // bs, ev).astype(np.float64)
        err = np.abs(g - ref)
        tol = ATOL + RTOL * np.abs(ref) + slack
        bad = err > tol
        assert not bad.any(), (b, int(bad.sum()), float((err / tol).max()), float(slack.max()))
        # away from the step the two agree far better than the stated tolerance
        assert err[slack == 0].max() <= 1e-4
        results.append((g, ref))
    return got, results


@pytest.mark.parametrize("kv,q", [("u8", "f16"), ("f16", "f16"), ("bf16", "bf16"), ("u8", "bf16")])
@pytest.mark.parametrize("D", [64, 128, 96, 256])
def test_diversity_matches_checker(pkg, kv, q, D):
    # areas: a multiple of 256 columns, tails of 32 / 96 columns, a sequence without a request, a single block
    lens = [700, 420, 333, 97, 1100]
    ev = [512, 288, 0, 32, 864]
    got, res = _run(pkg, kv, q, 8, 2, D, lens, 64, ev, seed=D + len(kv))
    assert len(res) == 4
    assert max(np.abs(r).max() for _, r in res) > 1.0


@pytest.mark.parametrize("kv,q,D,bs", [("u8", "f16", 80, 32), ("f16", "f16", 128, 16), ("bf16", "bf16", 64, 24), ("u8", "bf16", 192, 64),
                                       ("f16", "f16", 512, 16), ("u8", "f16", 128, 128), ("u8", "f16", 8, 32)])
def test_diversity_of_other_shapes(pkg, kv, q, D, bs):
    """Head sizes and block sizes the matrix-core kernels are not built for: the same output from the vector unit."""
    lens = [25 * bs + 7, 9 * bs + 1, 40, 3 * bs]
    ev = [20 * bs, 7 * bs, 0, bs]
    got, res = _run(pkg, kv, q, 8, 2, D, lens, 2 * bs, ev, seed=D + bs, bs=bs)
    assert len(res) == 3
    assert max(np.abs(r).max() for _, r in res) > 0.5


@pytest.mark.parametrize("kv,q,D", [("u8", "f16", 128), ("bf16", "bf16", 64), ("f16", "f16", 128), ("u8", "bf16", 96),
                                    ("f16", "f16", 256), ("u8", "f16", 256)])
def test_diversity_of_long_areas(pkg, kv, q, D):
    """Areas long enough for the launch that gives a workgroup four row blocks (the one the benchmark measures): a
    whole number of 128-row groups, an area whose last group holds one block and whose last 256 columns hold 32, and
    a short one beside them."""
    print(f"case diversity long {kv} D={D}", flush=True)
    lens = [4200, 2200, 500, 130]
    ev = [4096, 2080, 0, 96]
    got, res = _run(pkg, kv, q, 4, 2, D, lens, 32, ev, seed=31 + D)
    assert len(res) == 3


@pytest.mark.parametrize("Hkv", [1, 4, 8])
def test_diversity_over_kv_head_counts(pkg, Hkv):
    _run(pkg, "u8", "f16", 8, Hkv, 128, [600, 300], 32, [512, 256], seed=Hkv)


def test_identical_keys_closed_form(pkg):
    n, Hkv, D = 192, 2, 128
    keys = np.tile(np.linspace(-1.0, 1.0, Hkv * D).astype(np.float32), (n, 1))
    got, res = _run(pkg, "f16", "f16", 4, Hkv, D, [n], 32, [128], seed=1, keys=keys)
    g, _ = res[0]
    want = np.full((4, 128), -32.0)
    for rb in range(4):
        want[rb, rb * 32:(rb + 1) * 32] = -31.0
    np.testing.assert_allclose(g, want, rtol=0, atol=1e-3)


def test_diversity_is_deterministic(pkg):
    a, _ = _run(pkg, "u8", "f16", 8, 2, 128, [900, 500], 32, [832, 448], seed=9)
    b, _ = _run(pkg, "u8", "f16", 8, 2, 128, [900, 500], 32, [832, 448], seed=9)
    assert a.tobytes() == b.tobytes()


def test_diversity_rejects_bad_requests(pkg):
    import torch
    dev = torch.device("cuda:0")
    rng = np.random.default_rng(2)
    kc, ids, bib = RC.paged_key_cache(rng, [200], 2, 128, 32, "u8")
    op = pkg.PagedAttention(8, 2, 128, 32, "f16", "u8", num_layers=1, device=0)
    kc_d = torch.from_numpy(kc).to(dev)
    out = torch.zeros(4096, device=dev)
    with pytest.raises(pkg.PaError):  # no step yet
        op.adaptive_rkv_diversity(kc_d, 32, [64], out)
    op.step_begin(np.array([199], np.int32), np.array([0, 1], np.int32), bib)
    with pytest.raises(pkg.PaError):  # no block table for the layer yet
        op.adaptive_rkv_diversity(kc_d, 32, [64], out)
    op.set_block_indices(ids, kc.shape[0])
    with pytest.raises(pkg.PaError):  # not a multiple of the block size
        op.adaptive_rkv_diversity(kc_d, 32, [48], out)
    with pytest.raises(pkg.PaError):  # start not a multiple of the block size
        op.adaptive_rkv_diversity(kc_d, 16, [64], out)
    with pytest.raises(pkg.PaError):  # beyond the sequence's keys
        op.adaptive_rkv_diversity(kc_d, 32, [192], out)
    with pytest.raises(pkg.PaError):  # output too small: 4 x 128 values needed
        op.adaptive_rkv_diversity(kc_d, 32, [128], out[:500])
    assert list(op.adaptive_rkv_diversity(kc_d, 32, [0], out)) == [0, 0]  # nothing requested: nothing to do
    assert list(op.adaptive_rkv_diversity(kc_d, 32, [128], out)) == [0, 512]


def test_diversity_feeds_the_evictor(pkg):
    """The op's output goes to the evictor by device pointer, as in the pipeline: the evicted sets must equal those of
    the checker's evictor fed the same values."""
    import torch
    dev = torch.device("cuda:0")
    rng = np.random.default_rng(5)
    B, L, bs, Hkv, D = 2, 2, 32, 2, 128
    start, recent, mx = 32, 64, 352
    lens = [mx + 32, mx + 96]  # 1 and 3 blocks over
    kc, ids, bib = RC.paged_key_cache(rng, lens, Hkv, D, bs, "u8")
    op = pkg.PagedAttention(8, Hkv, D, bs, "f16", "u8", num_layers=L, device=0, stream=torch.cuda.current_stream(dev))
    op.step_begin((np.asarray(lens) - 1).astype(np.int32), np.arange(B + 1, dtype=np.int32), bib)
    op.set_block_indices(ids, kc.shape[0])
    kc_d = torch.from_numpy(kc).to(dev)
    cfg = pkg.CacheEvictionConfig(start, recent, mx, pkg.AggregationMode.ADAPTIVE_RKV, False, 0, None,
                                  pkg.AdaptiveRKVConfig(0.5, 8))
    ev = pkg.Evictor(cfg, bs, L, 7, max_sequences=B, max_tracked_tokens=1024, device=0,
                     stream=torch.cuda.current_stream(dev))
    refs = [O.CacheEvictionAlgorithm(start, recent, mx, O.MODE_ADAPTIVE_RKV, 0, bs, L, 7, attention_mass=0.5)
            for _ in range(B)]
    soff = np.concatenate([[0], np.cumsum(lens)]).astype(np.int64)
    layer_scores = [rng.random(int(soff[-1])).astype(np.float32) ** 3 for _ in range(L)]
    dev_scores = [torch.from_numpy(s).to(dev) for s in layer_scores]
    slots = np.arange(B, dtype=np.int32)
    ev.register_new_token_scores(slots, [t.data_ptr() for t in dev_scores], soff)
    for i in range(B):
        refs[i].register_new_token_scores([s[soff[i]:soff[i + 1]] for s in layer_scores])
    # the scheduler's evictable size: blocks * block_size - (max_cache_size - evictable_size)
    sizes = [int(-(-n // bs) * bs - (start + recent)) for n in lens]
    for i in range(B):
        b, e = refs[i].get_evictable_block_range(0)
        assert (e - b) * bs == sizes[i]
    total = sum((s // bs) * s for s in sizes)
    div = [torch.zeros(total, device=dev) for _ in range(L)]
    for l in range(L):
        doff = op.adaptive_rkv_diversity(kc_d, start, sizes, div[l], layer=l)
    op.synchronize()
    ev.register_block_diversity(slots, [t.data_ptr() for t in div], doff)
    host_div = [t.cpu().numpy() for t in div]
    for i in range(B):
        refs[i].register_block_diversity([d[doff[i]:doff[i + 1]] for d in host_div])
    got = ev.evict_logical_blocks(slots, max_blocks_per_entry=64)
    for i in range(B):
        exp = refs[i].evict_logical_blocks()
        assert got[i] == exp and len(exp[0]) == (lens[i] - mx) // bs
