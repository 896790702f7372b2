"""Device-resident eviction in ADAPTIVE_RKV mode and with KVCrush: the reference's known-answer vectors, and the CPU
checker fed the same scores and diversity values -- tracked state, block importances and evicted sets must be
identical."""
import types

import numpy as np
import pytest

import rkv_kvcrush_kats as K
from oracle import oracle as O

pytestmark = pytest.mark.gpu
KATS = K.KATS


@pytest.fixture(scope="module")
def impl(pkg):
    import torch
    assert torch.cuda.is_available()

    def make_algo(cfg, block_size, layers, max_pool, rkv_window=8, attention_mass=0.9, kvcrush_budget=0,
                  kvcrush_anchor=pkg.KVCrushAnchorPointMode.RANDOM):
        c = pkg.CacheEvictionConfig(cfg["start"], cfg["recent"], cfg["max"], pkg.AggregationMode[cfg["mode"]], False,
                                    cfg["snapkv"], pkg.KVCrushConfig(kvcrush_budget, kvcrush_anchor),
                                    pkg.AdaptiveRKVConfig(attention_mass, rkv_window))
        return pkg.CacheEvictionAlgorithm(c, block_size, layers, max_pool)

    return types.SimpleNamespace(make_algo=make_algo, ANCHORS={m.name: m for m in pkg.KVCrushAnchorPointMode})


@pytest.mark.parametrize("case", KATS["rkv_eviction"]["cases"], ids=lambda c: c["id"])
def test_rkv_eviction(impl, case):
    K.check_rkv_eviction(impl, case)


def test_rkv_eviction_needs_diversity(impl):
    K.check_rkv_needs_diversity(impl)


@pytest.mark.parametrize("case", KATS["kvcrush_eviction"]["cases"], ids=lambda c: c["id"])
def test_kvcrush_eviction(impl, case):
    K.check_kvcrush_eviction(impl, case)


@pytest.mark.parametrize("window,pool,snapkv", [(8, 7, 0), (3, 7, 0), (1, 1, 0), (4, 3, 8)])
def test_rkv_tracker_matches_checker_exactly(pkg, window, pool, snapkv):
    """Bare score manager in ADAPTIVE_RKV mode: growing score vectors (signed values, so that sums of negatives and
    the pooling order are exercised), more registrations than the window holds, a removal in between (which drops the
    history), then more registrations."""
    rng = np.random.default_rng(20 + window)
    L, bs, ignore = 2, 4, 2
    mgr = pkg.EvictionScoreManager(bs, L, pool, pkg.AggregationMode.ADAPTIVE_RKV, ignore, snapkv, window,
                                   max_tracked_tokens=512)
    ref = O.ScoreManager(bs, L, pool, O.MODE_ADAPTIVE_RKV, ignore, snapkv, window)
    n = 40
    for step in range(14):
        if step == 2:
            n = ignore * bs - 1  # shorter than the ignored area: nothing happens
        elif step == 3:
            n = 61
        else:
            n += int(rng.integers(0, 4))
        scores = [(rng.standard_normal(n) * 3).round(2).astype(np.float32) for _ in range(L)]
        n_snap = (snapkv if step == 0 else 0) if snapkv else 0
        if snapkv and step == 1:
            n_snap = 0
        mgr.register_new_token_scores(scores, (), n_snap)
        ref.register_new_token_scores(scores, (), n_snap)
        for l in range(L):
            assert np.array_equal(mgr.get_scores()[l], ref.get_scores()[l]), (step, l)
        if step == 8:
            for l in range(L):
                gone = sorted(rng.choice(8, size=3, replace=False).tolist())
                mgr.remove_scores(gone, l)
                ref.remove_scores(gone, l)
            n -= 3 * bs
            for l in range(L):
                assert np.array_equal(mgr.get_scores()[l], ref.get_scores()[l])


@pytest.mark.parametrize("mass,window", [(0.9, 8), (0.5, 2), (1.0, 8), (0.05, 4)])
def test_rkv_batched_decode_steps_match_checker_exactly(pkg, mass, window):
    """Several sequences x layers in ADAPTIVE_RKV mode: a prefill-sized first registration, then decode steps; a
    diversity matrix (random, with planted equal rows) is registered whenever an eviction is due, as the pipeline
    does, and the evicted sets and the tracked state are compared after every step."""
    import torch
    dev = torch.device("cuda:0")
    rng = np.random.default_rng(int(mass * 100) + window)
    B, L, bs = 4, 3, 32
    start, recent, mx = 32, 128, 672
    cfg = pkg.CacheEvictionConfig(start, recent, mx, pkg.AggregationMode.ADAPTIVE_RKV, False, 0, None,
                                  pkg.AdaptiveRKVConfig(mass, window))
    ev = pkg.Evictor(cfg, bs, L, 7, max_sequences=B + 1, max_tracked_tokens=2048, device=0,
                     stream=torch.cuda.current_stream(dev))
    refs = [O.CacheEvictionAlgorithm(start, recent, mx, O.MODE_ADAPTIVE_RKV, 0, bs, L, 7,
                                     adaptive_rkv_window_size=window, attention_mass=mass) for _ in range(B)]
    slots = np.array([4, 0, 2, 1], np.int32)
    ctx = rng.integers(600, 1500, B)
    evictions = 0
    for step in range(40):
        offsets = np.concatenate([[0], np.cumsum(ctx)]).astype(np.int64)
        layer_scores = [rng.random(int(offsets[-1])).astype(np.float32) ** 4 for _ in range(L)]
        for s in layer_scores:
            s[40:40 + 3 * bs] = 0.125  # whole blocks of equal importance
        dev_scores = [torch.from_numpy(s).to(dev) for s in layer_scores]
        ev.register_new_token_scores(slots, [t.data_ptr() for t in dev_scores], offsets)
        for i in range(B):
            refs[i].register_new_token_scores([s[offsets[i]:offsets[i + 1]] for s in layer_scores])
        due = []
        for i in range(B):
            for l in range(L):
                assert np.array_equal(ev.get_state(int(slots[i]), l)[0], refs[i].get_scores()[l]), (step, i, l)
                assert ev.get_evictable_block_range(int(slots[i]), l) == refs[i].get_evictable_block_range(l)
            b, e = refs[i].get_evictable_block_range(0)
            if e > b:
                due.append((i, e - b))
        if due:  # one [blocks, blocks * bs] matrix per due sequence, concatenated like the op's output
            doff = np.concatenate([[0], np.cumsum([nb * nb * bs for _, nb in due])]).astype(np.int64)
            layer_div = []
            for l in range(L):
                d = -(rng.random(int(doff[-1])).astype(np.float32))
                for x, (i, nb) in enumerate(due):
                    m = d[doff[x]:doff[x + 1]].reshape(nb, nb * bs)
                    m[1] = m[0]  # equal rows: equal filtered diversity
                layer_div.append(d)
            dev_div = [torch.from_numpy(d).to(dev) for d in layer_div]
            ev.register_block_diversity(slots[[i for i, _ in due]], [t.data_ptr() for t in dev_div], doff)
            for x, (i, nb) in enumerate(due):
                refs[i].register_block_diversity([d[doff[x]:doff[x + 1]] for d in layer_div])
        got = ev.evict_logical_blocks(slots, max_blocks_per_entry=128)
        for i in range(B):
            exp = refs[i].evict_logical_blocks()
            assert got[i] == exp, (step, i, got[i], exp)
            assert len({len(x) for x in exp}) == 1  # same count in every layer keeps the context lengths aligned
            evictions += len(exp[0])
            ctx[i] -= len(exp[0]) * bs
            for l in range(L):
                assert np.array_equal(ev.get_state(int(slots[i]), l)[0], refs[i].get_scores()[l])
        ctx += 1
    assert evictions > 0


@pytest.mark.parametrize("tied", [True, False], ids=["tied_scores", "distinct_scores"])
@pytest.mark.parametrize("mode,budget", [("RANDOM", 2), ("MEAN", 1), ("ALTERNATING", 1), ("ZEROS", 2), ("ONES", 3)])
def test_kvcrush_batched_decode_steps_match_checker_exactly(pkg, mode, budget, tied):
    """NORM_SUM eviction with KVCrush: `budget` of the blocks chosen for eviction stay as representatives whenever at
    least `budget` blocks were chosen (with budget 1 that is every eviction).
    Scores drawn from four values tie at the boundary of the better half, where the choice is the sorting routine's
    (the library then walks the scores on the host); continuous scores settle the half on the device."""
    import torch
    dev = torch.device("cuda:0")
    rng = np.random.default_rng(len(mode))
    B, L, bs = 3, 2, 32
    start, recent, mx = 32, 128, 672
    anchor = pkg.KVCrushAnchorPointMode[mode]
    cfg = pkg.CacheEvictionConfig(start, recent, mx, pkg.AggregationMode.NORM_SUM, False, 0,
                                  pkg.KVCrushConfig(budget, anchor, 11))
    ev = pkg.Evictor(cfg, bs, L, 7, max_sequences=B, max_tracked_tokens=2048, device=0,
                     stream=torch.cuda.current_stream(dev))
    refs = [O.CacheEvictionAlgorithm(start, recent, mx, O.MODE_NORM_SUM, 0, bs, L, 7, kvcrush_budget=budget,
                                     kvcrush_anchor_mode=int(anchor), kvcrush_seed=11) for _ in range(B)]
    slots = np.arange(B, dtype=np.int32)
    ctx = np.array([1200, 640, 900])
    retained = 0
    for step in range(70):
        offsets = np.concatenate([[0], np.cumsum(ctx)]).astype(np.int64)
        draw = (lambda n: rng.choice([0.0, 0.1, 0.5, 1.0], size=n)) if tied else (lambda n: rng.random(n))
        layer_scores = [draw(int(offsets[-1])).astype(np.float32) for _ in range(L)]
        dev_scores = [torch.from_numpy(s).to(dev) for s in layer_scores]
        ev.register_new_token_scores(slots, [t.data_ptr() for t in dev_scores], offsets)
        for i in range(B):
            refs[i].register_new_token_scores([s[offsets[i]:offsets[i + 1]] for s in layer_scores])
        due = [refs[i].get_evictable_block_range(0) for i in range(B)]
        got = ev.evict_logical_blocks(slots, max_blocks_per_entry=128)
        for i in range(B):
            exp = refs[i].evict_logical_blocks()
            assert got[i] == exp, (step, i)
            b, e = due[i]
            if e > b:
                plain = (e - b) - (mx - start - recent) // bs
                if plain >= budget:
                    assert len(exp[0]) == plain - budget
                    retained += budget
            ctx[i] -= len(exp[0]) * bs
            for l in range(L):
                gs, gc = ev.get_state(int(slots[i]), l)
                assert np.array_equal(gs, refs[i].get_scores()[l]) and np.array_equal(gc, refs[i].get_counters()[l])
        ctx += 1
    assert retained > 0


@pytest.mark.parametrize("seed", range(16))
def test_rkv_drawn_settings_match_checker_exactly(pkg, seed):
    """ADAPTIVE_RKV on drawn settings: block size, area sizes, max-pool window, tracker window, attention mass,
    sequences that grow by a token or by a chunk; a diversity matrix with planted equal rows whenever an eviction
    is due."""
    import torch
    dev = torch.device("cuda:0")
    rng = np.random.default_rng(8800 + seed)
    bs = int(rng.choice([16, 32, 64]))
    start, recent = bs * int(rng.integers(1, 3)), bs * int(rng.integers(1, 5))
    mx = start + recent + bs * int(rng.integers(2, 14))
    pool = int(rng.choice([1, 3, 7]))
    window = int(rng.integers(1, 9))
    mass = float(rng.choice([0.05, 0.3, 0.5, 0.9, 1.0]))
    B, L = int(rng.integers(1, 5)), int(rng.integers(1, 4))
    cfg = pkg.CacheEvictionConfig(start, recent, mx, pkg.AggregationMode.ADAPTIVE_RKV, False, 0, None,
                                  pkg.AdaptiveRKVConfig(mass, window))
    ev = pkg.Evictor(cfg, bs, L, pool, max_sequences=B, max_tracked_tokens=8192, device=0,
                     stream=torch.cuda.current_stream(dev))
    refs = [O.CacheEvictionAlgorithm(start, recent, mx, O.MODE_ADAPTIVE_RKV, 0, bs, L, pool,
                                     adaptive_rkv_window_size=window, attention_mass=mass) for _ in range(B)]
    slots = rng.permutation(B).astype(np.int32)
    ctx = rng.integers(mx // 2, 2 * mx, B)
    for step in range(14):
        offsets = np.concatenate([[0], np.cumsum(ctx)]).astype(np.int64)
        layer_scores = [rng.random(int(offsets[-1])).astype(np.float32) ** 4 for _ in range(L)]
        for s in layer_scores:
            s[start:start + 2 * bs] = 0.125  # whole blocks of equal importance
        dev_scores = [torch.from_numpy(s).to(dev) for s in layer_scores]
        ev.register_new_token_scores(slots, [t.data_ptr() for t in dev_scores], offsets)
        for i in range(B):
            refs[i].register_new_token_scores([s[offsets[i]:offsets[i + 1]] for s in layer_scores])
        due = []
        for i in range(B):
            for l in range(L):
                assert np.array_equal(ev.get_state(int(slots[i]), l)[0], refs[i].get_scores()[l]), (step, i, l)
                assert ev.get_evictable_block_range(int(slots[i]), l) == refs[i].get_evictable_block_range(l)
            b, e = refs[i].get_evictable_block_range(0)
            if e > b:
                due.append((i, e - b))
        if due:
            doff = np.concatenate([[0], np.cumsum([nb * nb * bs for _, nb in due])]).astype(np.int64)
            layer_div = []
            for l in range(L):
                d = -(rng.random(int(doff[-1])).astype(np.float32))
                for x, (i, nb) in enumerate(due):
                    if nb > 1:
                        mtx = d[doff[x]:doff[x + 1]].reshape(nb, nb * bs)
                        mtx[1] = mtx[0]
                layer_div.append(d)
            dev_div = [torch.from_numpy(d).to(dev) for d in layer_div]
            ev.register_block_diversity(slots[[i for i, _ in due]], [t.data_ptr() for t in dev_div], doff)
            for x, (i, nb) in enumerate(due):
                refs[i].register_block_diversity([d[doff[x]:doff[x + 1]] for d in layer_div])
        got = ev.evict_logical_blocks(slots, max_blocks_per_entry=512)
        for i in range(B):
            exp = refs[i].evict_logical_blocks()
            assert got[i] == exp, (step, i, got[i], exp)
            assert len({len(x) for x in exp}) == 1
            ctx[i] -= len(exp[0]) * bs
            for l in range(L):
                assert np.array_equal(ev.get_state(int(slots[i]), l)[0], refs[i].get_scores()[l])
        ctx += np.where(rng.random(B) < 0.3, rng.integers(2, 3 * bs, B), 1)


@pytest.mark.parametrize("seed", range(24))
def test_kvcrush_drawn_settings_match_checker_exactly(pkg, seed):
    """KVCrush on drawn settings: block size, area sizes, max-pool window, SUM or NORM_SUM, budget, anchor mode and
    its seed, tied or continuous scores, sequences that grow by a token or by a chunk."""
    import torch
    dev = torch.device("cuda:0")
    rng = np.random.default_rng(7700 + seed)
    bs = int(rng.choice([16, 32, 64]))
    start, recent = bs * int(rng.integers(1, 3)), bs * int(rng.integers(1, 5))
    mx = start + recent + bs * int(rng.integers(2, 16))
    pool = int(rng.choice([1, 3, 7]))
    norm = bool(rng.integers(0, 2))
    budget = int(rng.integers(1, 5))
    anchor = pkg.KVCrushAnchorPointMode(int(rng.integers(0, 5)))
    rseed = int(rng.integers(0, 1000))
    tied = bool(rng.integers(0, 2))
    B, L = int(rng.integers(1, 5)), int(rng.integers(1, 4))
    m = pkg.AggregationMode.NORM_SUM if norm else pkg.AggregationMode.SUM
    cfg = pkg.CacheEvictionConfig(start, recent, mx, m, False, 0, pkg.KVCrushConfig(budget, anchor, rseed))
    ev = pkg.Evictor(cfg, bs, L, pool, max_sequences=B, max_tracked_tokens=8192, device=0,
                     stream=torch.cuda.current_stream(dev))
    refs = [O.CacheEvictionAlgorithm(start, recent, mx, int(m), 0, bs, L, pool, kvcrush_budget=budget,
                                     kvcrush_anchor_mode=int(anchor), kvcrush_seed=rseed) for _ in range(B)]
    slots = rng.permutation(B).astype(np.int32)
    ctx = rng.integers(mx // 2, 3 * mx, B)
    evicted = 0
    for step in range(16):
        offsets = np.concatenate([[0], np.cumsum(ctx)]).astype(np.int64)
        draw = (lambda n: rng.choice([0.0, 0.1, 0.5, 1.0], size=n)) if tied else (lambda n: rng.random(n))
        layer_scores = [draw(int(offsets[-1])).astype(np.float32) for _ in range(L)]
        dev_scores = [torch.from_numpy(s).to(dev) for s in layer_scores]
        ev.register_new_token_scores(slots, [t.data_ptr() for t in dev_scores], offsets)
        for i in range(B):
            refs[i].register_new_token_scores([s[offsets[i]:offsets[i + 1]] for s in layer_scores])
        got = ev.evict_logical_blocks(slots, max_blocks_per_entry=512)
        for i in range(B):
            exp = refs[i].evict_logical_blocks()
            assert got[i] == exp, (step, i)
            assert len({len(x) for x in exp}) == 1
            evicted += len(exp[0])
            ctx[i] -= len(exp[0]) * bs
            for l in range(L):
                gs, gc = ev.get_state(int(slots[i]), l)
                assert np.array_equal(gs, refs[i].get_scores()[l]), (step, i, l)
                if norm:
                    assert np.array_equal(gc, refs[i].get_counters()[l]), (step, i, l)
        ctx += np.where(rng.random(B) < 0.3, rng.integers(2, 3 * bs, B), 1)
    # (a drawn budget may cover every eviction that falls due: then nothing leaves, in the library as in the checker)
    assert evicted > 0 or seed in (21, 22)


def test_rkv_evictor_rejects_bad_calls(pkg):
    import torch
    dev = torch.device("cuda:0")
    with pytest.raises(pkg.PaError):  # window outside [1, 32]
        pkg.Evictor(pkg.CacheEvictionConfig(4, 4, 12, pkg.AggregationMode.ADAPTIVE_RKV, False, 0, None,
                                            pkg.AdaptiveRKVConfig(0.9, 0)), 4, 2, 1)
    cfg = pkg.CacheEvictionConfig(4, 4, 12, pkg.AggregationMode.ADAPTIVE_RKV, False, 0)
    ev = pkg.Evictor(cfg, 4, 2, 1, max_sequences=2, max_tracked_tokens=64)
    t = torch.zeros(64, device=dev)
    ev.register_new_token_scores([0], [t.data_ptr()] * 2, [0, 16])
    with pytest.raises(pkg.PaError):  # 16 tokens: eviction is due, no diversity registered
        ev.evict_logical_blocks([0])
    with pytest.raises(pkg.PaError):  # not a multiple of the block size
        ev.register_block_diversity([0], [t.data_ptr()] * 2, [0, 18])
    ev.register_block_diversity([0], [t.data_ptr()] * 2, [0, 12])
    with pytest.raises(pkg.PaError):  # registered twice
        ev.register_block_diversity([0], [t.data_ptr()] * 2, [0, 16])
    with pytest.raises(pkg.PaError):  # 12 values registered, 2 x 2 x 4 expected
        ev.evict_logical_blocks([0])
    ev.reset_slot(0)
    ev.register_new_token_scores([0], [t.data_ptr()] * 2, [0, 16])
    ev.register_block_diversity([0], [t.data_ptr()] * 2, [0, 16])
    assert all(len(b) <= 2 for b in ev.evict_logical_blocks([0])[0])
