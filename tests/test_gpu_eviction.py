"""Device-resident score accumulation / eviction against the reference's known-answer vectors and against the CPU
checker fed the same scores: per-token state (f64 scores, u64 counters), block importances and evicted sets are
compared exactly."""
import types

import numpy as np
import pytest

import eviction_kats as K
from oracle import oracle as O

pytestmark = pytest.mark.gpu
KATS = K.KATS


@pytest.fixture(scope="module")
def impl(pkg):
    import torch
    assert torch.cuda.is_available()
    modes = {"SUM": pkg.AggregationMode.SUM, "NORM_SUM": pkg.AggregationMode.NORM_SUM}

    def score_manager(block_size, layers, max_pool, mode, ignore, snapkv, rkv_window):
        return pkg.EvictionScoreManager(block_size, layers, max_pool, mode, ignore, snapkv)

    def algo(start, recent, mx, mode, snapkv, block_size, layers, max_pool):
        cfg = pkg.CacheEvictionConfig(start, recent, mx, mode, False, snapkv)
        return pkg.CacheEvictionAlgorithm(cfg, block_size, layers, max_pool)

    return types.SimpleNamespace(ScoreManager=score_manager, CacheEvictionAlgorithm=algo, MODES=modes,
                                 snapkv_num_scores=pkg.snapkv_num_token_scores_to_aggregate)


def _no_skips(case):
    return all(not s["skips"] for s in case["steps"])


@pytest.mark.parametrize("case", [c for c in KATS["register_scores"]["cases"] if _no_skips(c)], ids=lambda c: c["id"])
def test_register_scores(impl, case):
    K.check_register_scores(impl, case, KATS["register_scores"]["abs_tol"])


@pytest.mark.parametrize("case", KATS["snapkv_counters"]["cases"], ids=lambda c: c["id"])
def test_snapkv_counters(impl, case):
    K.check_snapkv_counters(impl, case)


@pytest.mark.parametrize("case", [c for c in KATS["remove_scores"]["cases"] if _no_skips(c)], ids=lambda c: c["id"])
def test_remove_scores(impl, case):
    K.check_remove_scores(impl, case, KATS["remove_scores"]["abs_tol"])


@pytest.mark.parametrize("n", KATS["no_eviction_token_counts"]["counts"])
def test_no_eviction_below_total_size(impl, n):
    K.check_no_eviction_below_total_size(impl, n)


@pytest.mark.parametrize("case", KATS["range_calculation"]["cases"], ids=lambda c: str(c["num_tokens"]))
def test_evictable_range(impl, case):
    K.check_range(impl, case)


def test_starts_evicting_once_max_size_exceeded(impl):
    K.check_starts_evicting(impl)


@pytest.mark.parametrize("case", KATS["low_score_block_eviction"]["cases"], ids=lambda c: c["id"])
def test_low_score_blocks(impl, case):
    K.check_low_score(impl, case)


@pytest.mark.parametrize("case", KATS["normalization_setting"]["cases"],
                         ids=lambda c: f'{c["mode"]}_{c["power"]}_{"rising" if c["rising"] else "falling"}')
def test_normalization_setting(impl, case):
    K.check_normalization(impl, case)


@pytest.mark.parametrize("mode", KATS["scores_are_accumulated"]["modes"])
def test_scores_are_accumulated(impl, mode):
    K.check_scores_are_accumulated(impl, mode)


@pytest.mark.parametrize("c", KATS["invalid_config"]["algo_cases"])
def test_invalid_algo_config(pkg, c):
    cfg = pkg.CacheEvictionConfig(c["start"], c["recent"], c["max"], pkg.AggregationMode.NORM_SUM, False, 8)
    with pytest.raises(pkg.PaError):
        pkg.CacheEvictionAlgorithm(cfg, c["block_size"], c["layers"], 1)


@pytest.mark.parametrize("mode,snapkv", [("NORM_SUM", 0), ("NORM_SUM", 8), ("SUM", 0)])
def test_batched_decode_steps_match_checker_exactly(pkg, mode, snapkv):
    """Eviction settings of the scoring workload (start 32 / recent 128 / max 1024, block 32, max-pool 7): several
    sequences x layers, a prefill-sized first registration then 8 decode steps, evicting after each."""
    import torch
    dev = torch.device("cuda:0")
    rng = np.random.default_rng(4)
    B, L, bs = 5, 3, 32
    start, recent, mx = 32, 128, 1024
    m = pkg.AggregationMode[mode]
    ev = pkg.Evictor(pkg.CacheEvictionConfig(start, recent, mx, m, False, snapkv), bs, L, 7, max_sequences=B + 2,
                     max_tracked_tokens=4096, device=0, stream=torch.cuda.current_stream(dev))
    refs = [O.CacheEvictionAlgorithm(start, recent, mx, int(m), snapkv, bs, L, 7) for _ in range(B)]
    slots = np.array([6, 0, 3, 1, 4], np.int32)  # not the identity on purpose
    ctx = rng.integers(900, 2100, B)
    first = True
    for step in range(9):
        lens = ctx.copy()
        offsets = np.concatenate([[0], np.cumsum(lens)]).astype(np.int64)
        layer_scores = [rng.random(int(offsets[-1])).astype(np.float32) ** 3 for _ in range(L)]
        # plant exact ties: whole blocks of equal value
        for s in layer_scores:
            s[64:64 + 4 * bs] = 0.25
        dev_scores = [torch.from_numpy(s).to(dev) for s in layer_scores]
        n_snap = np.full(B, (snapkv if first else 1) if snapkv else 0, np.uint64)
        ev.register_new_token_scores(slots, [t.data_ptr() for t in dev_scores], offsets, n_snap)
        for i in range(B):
            refs[i].register_new_token_scores([s[offsets[i]:offsets[i + 1]] for s in layer_scores], (), int(n_snap[i]))
        for i in range(B):
            for l in range(L):
                gs, gc = ev.get_state(int(slots[i]), l)
                assert np.array_equal(gs, refs[i].get_scores()[l])
                if mode == "NORM_SUM":
                    assert np.array_equal(gc, refs[i].get_counters()[l])
                np.testing.assert_array_equal(ev.block_scores(int(slots[i]), l), refs[i].block_scores(l))
                assert ev.get_evictable_block_range(int(slots[i]), l) == refs[i].get_evictable_block_range(l)
        got = ev.evict_logical_blocks(slots, max_blocks_per_entry=256)
        for i in range(B):
            exp = refs[i].evict_logical_blocks()
            assert got[i] == exp, (step, i)
            ctx[i] -= len(exp[0]) * bs
            for l in range(L):
                gs, gc = ev.get_state(int(slots[i]), l)
                assert np.array_equal(gs, refs[i].get_scores()[l])
                if mode == "NORM_SUM":
                    assert np.array_equal(gc, refs[i].get_counters()[l])
        ctx += 1
        first = False
    assert any(len(b) for b in got[0]) or True


@pytest.mark.parametrize("seed", range(40))
def test_random_eviction_settings_match_checker_exactly(pkg, seed):
    """Drawn settings instead of the scoring workload's: block size, area sizes, max-pool window, aggregation mode,
    SnapKV window, sequences that grow by one token or by a chunk per step, planted ties; state, block scores,
    ranges and evicted blocks equal to the checker's after every step."""
    import torch
    dev = torch.device("cuda:0")
    rng = np.random.default_rng(9000 + seed)
    bs = int(rng.choice([16, 32, 64]))
    start, recent = bs * int(rng.integers(1, 4)), bs * int(rng.integers(1, 6))
    mx = start + recent + bs * int(rng.integers(1, 20))
    pool = int(rng.choice([1, 3, 7]))
    mode = ["SUM", "NORM_SUM"][int(rng.integers(0, 2))]
    snapkv = int(rng.choice([0, 0, 4, 8]))
    B, L = int(rng.integers(1, 7)), int(rng.integers(1, 4))
    m = pkg.AggregationMode[mode]
    ev = pkg.Evictor(pkg.CacheEvictionConfig(start, recent, mx, m, False, snapkv), bs, L, pool, max_sequences=B,
                     max_tracked_tokens=8192, device=0, stream=torch.cuda.current_stream(dev))
    refs = [O.CacheEvictionAlgorithm(start, recent, mx, int(m), snapkv, bs, L, pool) for _ in range(B)]
    slots = rng.permutation(B).astype(np.int32)
    ctx = rng.integers(max(snapkv, 1), 3 * mx, B)   # some sequences start below the budget, some far above
    first, total = True, 0
    for step in range(10):
        offsets = np.concatenate([[0], np.cumsum(ctx)]).astype(np.int64)
        layer_scores = [rng.random(int(offsets[-1])).astype(np.float32) ** 3 for _ in range(L)]
        for s in layer_scores:   # ties: runs of equal values, and exact zeros
            a = int(rng.integers(0, max(1, len(s) - 3 * bs)))
            s[a:a + 3 * bs] = 0.25
            s[rng.random(len(s)) < 0.05] = 0.0
        dev_scores = [torch.from_numpy(s).to(dev) for s in layer_scores]
        n_snap = np.full(B, (snapkv if first else 1) if snapkv else 0, np.uint64)
        ev.register_new_token_scores(slots, [t.data_ptr() for t in dev_scores], offsets, n_snap)
        for i in range(B):
            refs[i].register_new_token_scores([s[offsets[i]:offsets[i + 1]] for s in layer_scores], (), int(n_snap[i]))
        for i in range(B):
            for l in range(L):
                gs, gc = ev.get_state(int(slots[i]), l)
                assert np.array_equal(gs, refs[i].get_scores()[l]), (step, i, l)
                if mode == "NORM_SUM":
                    assert np.array_equal(gc, refs[i].get_counters()[l]), (step, i, l)
                np.testing.assert_array_equal(ev.block_scores(int(slots[i]), l), refs[i].block_scores(l))
                assert ev.get_evictable_block_range(int(slots[i]), l) == refs[i].get_evictable_block_range(l)
        got = ev.evict_logical_blocks(slots, max_blocks_per_entry=512)
        for i in range(B):
            exp = refs[i].evict_logical_blocks()
            assert got[i] == exp, (step, i)
            total += len(exp[0])
            ctx[i] -= len(exp[0]) * bs
            for l in range(L):
                gs, gc = ev.get_state(int(slots[i]), l)
                assert np.array_equal(gs, refs[i].get_scores()[l]), (step, i, l)
                if mode == "NORM_SUM":
                    assert np.array_equal(gc, refs[i].get_counters()[l]), (step, i, l)
        ctx += np.where(rng.random(B) < 0.3, rng.integers(2, 3 * bs, B), 1)   # a decode token, or a chunk
        first = False
    assert total > 0 or int(ctx.max()) <= mx + bs


@pytest.mark.parametrize("mode", ["NORM_SUM", "ADAPTIVE_RKV"])
def test_scores_may_be_rewritten_in_stream_order_right_after_registering(pkg, mode):
    """pa_evictor_register_scores returns with its kernel queued: the score tensors are read in stream order, so work
    queued behind the call on the same stream -- here a fill that overwrites them at once, many times over a large
    registration -- must not reach what the registration reads."""
    import torch
    dev = torch.device("cuda:0")
    rng = np.random.default_rng(77)
    B, L, bs = 6, 4, 32
    m = pkg.AggregationMode[mode]
    rkv = {"adaptive_rkv_window_size": 4, "attention_mass": 0.9} if mode == "ADAPTIVE_RKV" else {}
    cfg = (pkg.CacheEvictionConfig(32, 128, 1024, m, False, 0, None, pkg.AdaptiveRKVConfig(0.9, 4)) if rkv else
           pkg.CacheEvictionConfig(32, 128, 1024, m, False, 0))
    ev = pkg.Evictor(cfg, bs, L, 7, max_sequences=B, max_tracked_tokens=40000, device=0,
                     stream=torch.cuda.current_stream(dev))
    refs = [O.CacheEvictionAlgorithm(32, 128, 1024, int(m), 0, bs, L, 7, **rkv) for _ in range(B)]
    slots = np.arange(B, dtype=np.int32)
    lens = rng.integers(30000, 36000, B)
    offsets = np.concatenate([[0], np.cumsum(lens)]).astype(np.int64)
    bufs = [torch.empty(int(offsets[-1]), dtype=torch.float32, device=dev) for _ in range(L)]
    for step in range(4):
        host = [rng.random(int(offsets[-1])).astype(np.float32) for _ in range(L)]
        for t, h in zip(bufs, host):
            t.copy_(torch.from_numpy(h).to(dev))
        ev.register_new_token_scores(slots, [t.data_ptr() for t in bufs], offsets, None)
        for t in bufs:  # queued behind the registration on the same stream, no synchronisation in between
            t.fill_(float("nan"))
        for i in range(B):
            refs[i].register_new_token_scores([h[offsets[i]:offsets[i + 1]] for h in host], (), 0)
    for i in range(B):
        for l in range(L):
            gs, gc = ev.get_state(i, l)
            assert np.array_equal(gs, refs[i].get_scores()[l]), (i, l)


def test_evictor_rejects_bad_calls(pkg):
    import torch
    ev = pkg.Evictor(pkg.CacheEvictionConfig(32, 32, 192, pkg.AggregationMode.NORM_SUM, False, 4), 4, 2, 1,
                     max_sequences=2, max_tracked_tokens=256)
    t = torch.zeros(300, device="cuda:0")
    with pytest.raises(pkg.PaError):  # slot out of range
        ev.register_new_token_scores([2], [t.data_ptr()] * 2, [0, 10], [1])
    with pytest.raises(pkg.PaError):  # more SnapKV scores than the window
        ev.register_new_token_scores([0], [t.data_ptr()] * 2, [0, 50], [5])
    with pytest.raises(pkg.PaError):  # longer than max_tracked_tokens
        ev.register_new_token_scores([0], [t.data_ptr()] * 2, [0, 300], [1])
    ev.register_new_token_scores([0], [t.data_ptr()] * 2, [0, 100], [4])
    with pytest.raises(pkg.PaError):  # scores may not shrink
        ev.register_new_token_scores([0], [t.data_ptr()] * 2, [0, 60], [1])
    ev.reset_slot(0)
    assert ev.get_state(0, 0)[0].size == 0


def test_decode_scores_feed_eviction_like_the_pipeline(pkg):
    """The scoring workload's loop at reduced size: decode step -> scores.<L> on the device -> register -> evict ->
    drop the evicted blocks from the block table -> next step.  The checker's eviction restatement is fed the same
    device scores; evicted sets and tracked state must be identical, and the attention itself stays within tolerance
    of the checker on the shrinking cache."""
    import torch
    import harness as H
    dev = torch.device("cuda:0")
    rng = np.random.default_rng(1004)
    B, Hq, Hkv, D, bs, L = 3, 8, 2, 128, 32, 2
    start, recent, mx = 32, 128, 1024
    cfg = pkg.CacheEvictionConfig(start, recent, mx, pkg.AggregationMode.NORM_SUM, False, 0)
    ev = pkg.Evictor(cfg, bs, L, 7, max_sequences=B, max_tracked_tokens=4096, device=0,
                     stream=torch.cuda.current_stream(dev))
    refs = [O.CacheEvictionAlgorithm(start, recent, mx, O.MODE_NORM_SUM, 0, bs, L, 7) for _ in range(B)]
    ctx0 = np.array([1100, 1500, 1043])
    case = H.build_case(H.case_from_lens("evict_flow", Hq, Hkv, D, bs, "f16", "u8", ctx0, np.ones(B, int)), 1004,
                        outliers=True, pool_factor=1.5)
    op = pkg.PagedAttention(Hq, Hkv, D, bs, "f16", "u8", num_layers=L, device=0, stream=torch.cuda.current_stream(dev))
    kc = [torch.from_numpy(case["key_cache0"]).to(dev) for _ in range(L)]
    vc = [torch.from_numpy(case["value_cache0"]).to(dev) for _ in range(L)]
    kc_h = [case["key_cache0"].copy() for _ in range(L)]
    vc_h = [case["value_cache0"].copy() for _ in range(L)]
    # per layer, per sequence block tables (they diverge once layers evict different blocks)
    tables = [[list(case["block_indices"][case["block_indices_begins"][b]:case["block_indices_begins"][b + 1]])
               for b in range(B)] for _ in range(L)]
    free = [p for p in range(case["num_blocks"]) if p not in set(case["block_indices"].tolist())]
    past = ctx0.copy()
    evicted_any = False
    for step in range(10):
        T = B
        q = H.O.to_bits(rng.standard_normal((T, Hq * D)).astype(np.float32), H.O.DT_F16)
        k = H.O.to_bits(rng.standard_normal((T, Hkv * D)).astype(np.float32), H.O.DT_F16)
        v = H.O.to_bits(rng.standard_normal((T, Hkv * D)).astype(np.float32), H.O.DT_F16)
        for l in range(L):  # room for the new token
            for b in range(B):
                if (past[b] + 1 + bs - 1) // bs > len(tables[l][b]):
                    tables[l][b].append(free.pop())
        sb = np.arange(B + 1, dtype=np.int32)
        op.step_begin(past.astype(np.int32), sb, np.concatenate([[0], np.cumsum([len(t) for t in tables[0]])]))
        qd, kd, vd = (H.to_device_16(torch, x, "f16", dev) for x in (q, k, v))
        scores = []
        for l in range(L):
            bib = np.concatenate([[0], np.cumsum([len(t) for t in tables[l]])]).astype(np.int32)
            ids = np.concatenate(tables[l]).astype(np.int32)
            op.set_block_indices(ids, case["num_blocks"], layer=l)
            out = torch.zeros_like(qd)
            sc = torch.zeros(op.total_scores, dtype=torch.float32, device=dev)
            op.forward(qd, kd, vd, kc[l], vc[l], out, sc, layer=l)
            scores.append(sc)
            # checker on the same tables
            H.O.kv_append(k, v, H.O.DT_F16, kc_h[l], vc_h[l], H.O.DT_U8, past.astype(np.int32), sb, ids, bib, Hkv, D, bs)
            ro, _, rs = H.O.paged_attention(q, H.O.DT_F16, kc_h[l], vc_h[l], H.O.DT_U8, past.astype(np.int32), sb, ids,
                                            bib, Hq, Hkv, D, bs, 1.0 / np.sqrt(D), 0, None, True, 8)
            op.synchronize()
            H.assert_close(out.float().cpu().numpy(), ro, "f16")
            H.assert_close(sc.cpu().numpy(), rs, "f16", "scores")
            assert np.array_equal(kc[l].cpu().numpy(), kc_h[l])
        offsets = np.concatenate([[0], np.cumsum(past + 1)]).astype(np.int64)
        ev.register_new_token_scores(np.arange(B), [s.data_ptr() for s in scores], offsets, None)
        host_scores = [s.cpu().numpy() for s in scores]
        for b in range(B):
            refs[b].register_new_token_scores([hs[offsets[b]:offsets[b + 1]] for hs in host_scores])
        got = ev.evict_logical_blocks(np.arange(B), max_blocks_per_entry=128)
        n_ev = np.zeros(B, int)
        for b in range(B):
            exp = refs[b].evict_logical_blocks()
            assert got[b] == exp, (step, b)
            assert len({len(e) for e in exp}) == 1  # every layer evicts the same number of blocks
            n_ev[b] = len(exp[0])
            for l in range(L):
                for blk in sorted(exp[l], reverse=True):
                    free.append(tables[l][b].pop(blk))
                gs, gc = ev.get_state(b, l)
                assert np.array_equal(gs, refs[b].get_scores()[l]) and np.array_equal(gc, refs[b].get_counters()[l])
        evicted_any = evicted_any or n_ev.any()
        past = past + 1 - n_ev * bs
    assert evicted_any
    assert all(p <= mx + bs for p in past)  # per-sequence cache stays capped (cache_eviction.cpp:297-303)


@pytest.mark.parametrize("snapkv", [0, 8])
def test_full_size_scoring_workload_eviction_matches_checker(pkg, snapkv):
    """The scoring workload at full size: 256 sequences at 8192 tokens of context (Llama-3-8B shape, u8 KV, two
    layers with their own caches and tables), real decode scores on the device -> register -> evict -> drop the
    evicted blocks from the tables, for 34 consecutive steps (NORM_SUM, start 32 / recent 128 / max 1024, max-pool 7).
    The checker's restatement of CacheEvictionAlgorithm is fed the same device scores: evicted lists, f64 scores and
    u64 counters must be identical.  The first eviction frees 224 blocks per (sequence, layer); the second one
    comes 31 steps later."""
    import torch
    dev = torch.device("cuda:0")
    B, Hq, Hkv, D, bs, L = 256, 32, 8, 128, 32, 2
    start, recent, mx = 32, 128, 1024
    ctx0 = 8192
    gen = torch.Generator(device=dev).manual_seed(1004 + snapkv)
    rng = np.random.default_rng(1004 + snapkv)
    nblk0 = ctx0 // bs + 1
    pool = B * (nblk0 + 1)
    caches = []
    for l in range(L):
        pair = []
        for _ in range(2):
            c = torch.randint(0, 256, (pool, Hkv, bs, D + 8), dtype=torch.uint8, device=dev, generator=gen)
            hdr = torch.empty(pool, Hkv, bs, 2, dtype=torch.float32, device=dev)
            hdr[..., 0] = 0.02 + 0.04 * torch.rand(pool, Hkv, bs, device=dev, generator=gen)
            hdr[..., 1] = 100.0 + 50.0 * torch.rand(pool, Hkv, bs, device=dev, generator=gen)
            c[..., :8] = hdr.view(torch.uint8).view(pool, Hkv, bs, 8)
            pair.append(c)
            del hdr
        caches.append(pair)
    perm = rng.permutation(pool)
    tables = [[list(perm[b * (nblk0 + 1): b * (nblk0 + 1) + nblk0]) for b in range(B)] for _ in range(L)]
    # one more block per sequence and layer, for growth; like the reference's allocator, every layer has a free list
    # of its own (a block freed by layer l's eviction is only ever handed back to layer l)
    spare = [[[int(perm[b * (nblk0 + 1) + nblk0])] for b in range(B)] for _ in range(L)]
    cfg = pkg.CacheEvictionConfig(start, recent, mx, pkg.AggregationMode.NORM_SUM, False, snapkv)
    ev = pkg.Evictor(cfg, bs, L, 7, max_sequences=B, max_tracked_tokens=ctx0 + 64, device=0,
                     stream=torch.cuda.current_stream(dev))
    refs = [O.CacheEvictionAlgorithm(start, recent, mx, O.MODE_NORM_SUM, snapkv, bs, L, 7) for _ in range(B)]
    op = pkg.PagedAttention(Hq, Hkv, D, bs, "f16", "u8", num_layers=L, device=0, stream=torch.cuda.current_stream(dev))
    past = np.full(B, ctx0, np.int64)
    slots = np.arange(B, dtype=np.int32)
    sb = np.arange(B + 1, dtype=np.int32)
    evictions = []
    for step in range(34):
        for b in range(B):
            if (past[b] + 1 + bs - 1) // bs > len(tables[0][b]):
                for l in range(L):
                    tables[l][b].append(spare[l][b].pop())
        q = torch.randn(B, Hq * D, device=dev, generator=gen).to(torch.float16)
        k = torch.randn(B, Hkv * D, device=dev, generator=gen).to(torch.float16)
        v = torch.randn(B, Hkv * D, device=dev, generator=gen).to(torch.float16)
        bib = np.concatenate([[0], np.cumsum([len(t) for t in tables[0]])]).astype(np.int32)
        op.step_begin(past.astype(np.int32), sb, bib)
        scores = []
        for l in range(L):
            assert [len(t) for t in tables[l]] == [len(t) for t in tables[0]]
            op.set_block_indices(np.concatenate(tables[l]).astype(np.int32), pool, layer=l)
            out = torch.empty_like(q)
            sc = torch.full((op.total_scores,), float("nan"), dtype=torch.float32, device=dev)
            op.forward(q, k, v, caches[l][0], caches[l][1], out, sc, layer=l)
            scores.append(sc)
        op.synchronize()
        offsets = np.concatenate([[0], np.cumsum(past + 1)]).astype(np.int64)
        n_snap = np.full(B, 1 if snapkv else 0, np.uint64)   # generation phase: one score row per step
        ev.register_new_token_scores(slots, [s.data_ptr() for s in scores], offsets, n_snap)
        host = [s.cpu().numpy() for s in scores]
        assert all(np.isfinite(h).all() for h in host)
        for b in range(B):
            refs[b].register_new_token_scores([h[offsets[b]:offsets[b + 1]] for h in host], (), int(n_snap[b]))
        check_all = step in (0, 1, 7, 31, 32)
        for b in (range(B) if check_all else (0, 97, 255)):
            for l in range(L):
                gs, gc = ev.get_state(b, l)
                assert np.array_equal(gs, refs[b].get_scores()[l]), (step, b, l)
                assert np.array_equal(gc, refs[b].get_counters()[l]), (step, b, l)
        got = ev.evict_logical_blocks(slots, max_blocks_per_entry=256)
        n_ev = np.zeros(B, np.int64)
        for b in range(B):
            exp = refs[b].evict_logical_blocks()
            assert got[b] == exp, (step, b)
            n_ev[b] = len(exp[0])
            for l in range(L):
                assert len(exp[l]) == n_ev[b]
                for blk in sorted(exp[l], reverse=True):
                    spare[l][b].append(int(tables[l][b].pop(blk)))
        if step in (0, 31):
            for b in range(0, B, 17):
                for l in range(L):
                    gs, gc = ev.get_state(b, l)
                    assert np.array_equal(gs, refs[b].get_scores()[l]) and np.array_equal(gc, refs[b].get_counters()[l])
        evictions.append(n_ev.copy())
        past = past + 1 - n_ev * bs
    assert (evictions[0] == 224).all()            # 251 evictable blocks, 27 kept
    # then one token per step: 1025 + k tokens at step k pass max_cache_size + block_size - 1 = 1055 at k = 31
    assert all((e == 0).all() for e in evictions[1:31])
    assert (evictions[31] == 1).all() and (evictions[32] == 0).all() and (evictions[33] == 0).all()
    assert (past <= mx + bs).all()
