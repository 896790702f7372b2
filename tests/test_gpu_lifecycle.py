"""Handles of the C-ABI over a long-running process: contexts, evictors and caches that are created, used and
destroyed again and again give the device's memory back, and contexts of different shapes used in turn on one
device do not disturb each other (each gives the bits it gives alone)."""
import gc

import numpy as np
import pytest

import harness as H

pytestmark = pytest.mark.gpu

SHAPES = [  # Hq, Hkv, D, bs, q, kv, past, new
    (8, 2, 128, 32, "f16", "u8", [700, 64, 9000], [1, 1, 1]),          # u8 decode kernel, several splits
    (12, 4, 96, 32, "f16", "f16", [300, 40, 0], [1, 1, 70]),           # matrix kernel beside the 16-bit decode kernel
    (4, 2, 64, 16, "bf16", "bf16", [100, 5000], [1, 1]),               # 16-bit decode kernel
    (16, 8, 256, 32, "bf16", "u8", [0, 1200], [130, 1]),               # u8 chunk + decode on two streams
    (6, 2, 80, 32, "f16", "u8", [500, 33], [1, 9]),                    # shape-generic kernels
]


def _cases():
    return [H.build_case(H.case_from_lens(f"life{i}", Hq, Hkv, D, bs, q, kv, past, new), seed=300 + i)
            for i, (Hq, Hkv, D, bs, q, kv, past, new) in enumerate(SHAPES)]


def _cycle(pkg, torch, dev, case):
    """One context, one evictor and one cache: created, used for a step, destroyed."""
    r = H.run_case_on_gpu(pkg, case, dev)
    layers = 2
    cfg = pkg.CacheEvictionConfig(case["bs"], 2 * case["bs"], 6 * case["bs"], pkg.AggregationMode.NORM_SUM, False, 0)
    ev = pkg.Evictor(cfg, case["bs"], layers, 7, max_sequences=len(case["past_lens"]), max_tracked_tokens=16384,
                     device=0, stream=torch.cuda.current_stream(dev))
    scores = torch.from_numpy(r["scores"]).to(dev)
    kv_lens = case["past_lens"] + case["new_lens"]
    offsets = np.concatenate([[0], np.cumsum(kv_lens)]).astype(np.int64)
    slots = np.arange(len(kv_lens), dtype=np.int32)
    ev.register_new_token_scores(slots, [scores.data_ptr()] * layers, offsets)
    evicted = ev.evict_logical_blocks(slots)
    cache = pkg.KVCacheManager(layers, case["Hkv"], case["D"], case["bs"], case["kv_dtype"], device=0)
    cache.allocate_cache_if_needed(48)
    cache.allocate_cache_if_needed(96)
    cache.copy_blocks({1: [50, 51], 2: [52]})
    torch.cuda.synchronize(dev)
    n_evicted = sum(len(b) for seq in evicted for b in seq)
    out16 = r["out16"]
    r["op"] = None
    del r, ev, cache, scores
    gc.collect()
    return out16, n_evicted


def test_handles_created_and_destroyed_in_a_loop_return_their_memory(pkg):
    import torch
    dev = torch.device("cuda:0")
    cases = _cases()
    first = [_cycle(pkg, torch, dev, c) for c in cases]  # warm: device code uploaded, torch's pools at size
    assert any(n for _, n in first)                      # some sequence was over its budget: the evictor did work
    torch.cuda.synchronize(dev)
    torch.cuda.empty_cache()
    free0 = torch.cuda.mem_get_info(dev)[0]
    for rep in range(12):
        for i, c in enumerate(cases):
            out16, n = _cycle(pkg, torch, dev, c)
            assert np.array_equal(out16, first[i][0]), (rep, c["name"])
            assert n == first[i][1], (rep, c["name"])
    torch.cuda.synchronize(dev)
    torch.cuda.empty_cache()
    free1 = torch.cuda.mem_get_info(dev)[0]
    # 60 contexts, evictors and caches later: what a leaked workspace, staging area or cache piece would take
    # (each of them megabytes) is not missing
    assert free0 - free1 < (1 << 20), (free0, free1)


def test_contexts_of_different_shapes_used_in_turn_give_the_bits_they_give_alone(pkg):
    import torch
    dev = torch.device("cuda:0")
    cases = _cases()
    alone = [H.run_case_on_gpu(pkg, c, dev) for c in cases]
    ops = [a["op"] for a in alone]
    for rnd in range(3):  # every context steps again, in turn, on the workspaces it kept
        order = range(len(cases)) if rnd % 2 == 0 else reversed(range(len(cases)))
        for i in order:
            again = H.run_case_on_gpu(pkg, cases[i], dev, op=ops[i])
            for what in ("out16", "scores", "key_cache", "value_cache"):
                assert np.array_equal(again[what], alone[i][what], equal_nan=what == "scores"), (rnd, cases[i]["name"], what)
    want = H.run_case_on_checker(cases[0])
    H.assert_close(alone[0]["out"], want["out"], cases[0]["q_dtype"])


def test_two_host_threads_each_with_contexts_and_a_stream_of_their_own(pkg):
    """The library keeps no state outside its handles (error texts of handle-less calls are per thread): two host
    threads that create, use and destroy contexts at the same time, each on its own stream, get the bits a single
    thread gets."""
    import threading
    import torch
    dev = torch.device("cuda:0")
    cases = _cases()
    alone = [H.run_case_on_gpu(pkg, c, dev) for c in cases]
    for a in alone:
        a["op"] = None
    problems = []

    def worker(k):
        try:
            s = torch.cuda.Stream(dev)
            with torch.cuda.stream(s):
                for rep in range(5):
                    order = list(range(len(cases)))
                    if k:
                        order.reverse()
                    for i in order:
                        r = H.run_case_on_gpu(pkg, cases[i], dev)
                        for what in ("out16", "scores", "key_cache", "value_cache"):
                            if not np.array_equal(r[what], alone[i][what]):
                                problems.append((k, rep, cases[i]["name"], what))
                        r["op"] = None
        except BaseException as e:  # noqa: BLE001 -- reported by the main thread
            problems.append((k, repr(e)))

    threads = [threading.Thread(target=worker, args=(k,)) for k in range(2)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not problems, problems[:5]
