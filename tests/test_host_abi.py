"""CPU-side checks of the product: the C-ABI library loads and exports what include/pa_amd.h declares, and its
host-only entry points (step packing, SnapKV window, block-count normalisation, config validation) agree with the
CPU checker and the reference's vectors.  No GPU compute here."""
import ctypes as C
import os
import re

import numpy as np
import pytest

import eviction_kats as K
from oracle import oracle as O

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_library_exports_every_declared_symbol(pkg):
    header = open(os.path.join(ROOT, "include", "pa_amd.h")).read()
    header = re.sub(r"/\*.*?\*/", "", header, flags=re.S)
    declared = set(re.findall(r"\b(pa_[a-z0-9_]+)\s*\(", header))
    lib_mod = __import__("openvino_genai_amd._lib", fromlist=["x"])
    assert declared == set(lib_mod.EXPORTS)
    so = C.CDLL(lib_mod.SO_PATH)
    for name in declared:
        assert hasattr(so, name), name
    assert b"gfx950" in pkg.lib().pa_version()


def test_pack_step_matches_checker(pkg):
    rng = np.random.default_rng(0)
    for _ in range(20):
        B = int(rng.integers(1, 40))
        bs = int(rng.choice([16, 32]))
        evicted = rng.integers(0, 4, B) * bs
        processed = evicted + rng.integers(0, 5000, B)
        scheduled = rng.integers(1, 600, B)
        nblk = (processed - evicted + scheduled + bs - 1) // bs
        skipped = np.minimum(rng.integers(0, 3, B), (processed - evicted) // bs)
        got = pkg.pack_step(processed, evicted, skipped, scheduled, nblk, bs)
        ref = O.pack_step(processed, evicted, skipped, scheduled, nblk, bs)
        for g, r in zip(got, ref):
            assert np.array_equal(g, r)


def test_pack_step_rejects_bad_input(pkg):
    with pytest.raises(pkg.PaError) as e:
        pkg.pack_step([10], [32], [0], [1], [1], 32)  # more evicted than processed
    assert e.value.status == -6


@pytest.mark.parametrize("case", K.KATS["snapkv_score_aggregator"]["cases"], ids=lambda c: c["id"])
def test_snapkv_window_vectors(pkg, case):
    assert pkg.snapkv_num_token_scores_to_aggregate(case["snapkv"], case["prompt_len"], case["num_scheduled"],
                                                    case["num_processed"]) == case["ref"]


def test_snapkv_window_matches_checker(pkg):
    rng = np.random.default_rng(1)
    for _ in range(300):
        a = [int(v) for v in rng.integers(0, 200, 4)]
        assert pkg.snapkv_num_token_scores_to_aggregate(*a) == O.snapkv_num_scores(*a)


def test_normalize_num_kv_blocks_matches_checker(pkg):
    rng = np.random.default_rng(2)
    for _ in range(100):
        nb = int(rng.choice([0, 0, 123, 5000]))
        gib = int(rng.choice([0, 1, 3, 8]))
        bs = int(rng.choice([16, 32]))
        bb = int(rng.integers(1 << 12, 1 << 22))
        total = int(rng.choice([1 << 32, 1 << 40]))
        try:
            ref = O.normalize_num_kv_blocks(nb, gib, bs, bb, total)
        except RuntimeError:
            with pytest.raises(pkg.PaError):
                pkg.normalize_num_kv_blocks(nb, gib, bs, bb, total)
            continue
        assert pkg.normalize_num_kv_blocks(nb, gib, bs, bb, total) == ref


def test_config_surface_keeps_reference_names(pkg):
    # src/python/py_continuous_batching_pipeline.cpp:344-466 of the reference
    assert [m.name for m in pkg.AggregationMode] == ["SUM", "NORM_SUM", "ADAPTIVE_RKV"]
    cfg = pkg.CacheEvictionConfig()
    assert (cfg.get_start_size(), cfg.get_recent_size(), cfg.get_max_cache_size(), cfg.get_evictable_size()) == (32, 128, 672, 512)
    assert cfg.aggregation_mode == pkg.AggregationMode.NORM_SUM and cfg.snapkv_window_size == 8 and not cfg.apply_rotation
    for name in ("aggregation_mode", "apply_rotation", "snapkv_window_size", "get_start_size", "get_recent_size",
                 "get_max_cache_size", "get_evictable_size", "to_string"):
        assert hasattr(cfg, name)
    sc = pkg.SchedulerConfig()
    for name, default in (("max_num_batched_tokens", 256), ("num_kv_blocks", 0), ("cache_size", 0),
                          ("dynamic_split_fuse", True), ("use_cache_eviction", False), ("max_num_seqs", 256),
                          ("enable_prefix_caching", False), ("use_sparse_attention", False)):
        assert getattr(sc, name) == default
    assert "use_cache_eviction: false" in sc.to_string()
    # SparseAttentionMode / SparseAttentionConfig: py_continuous_batching_pipeline.cpp:412-440,
    # include/openvino/genai/sparse_attention.hpp:10-83
    assert [m.name for m in pkg.SparseAttentionMode] == ["TRISHAPE", "XATTENTION"]
    sp = sc.sparse_attention_config
    for name, default in (("mode", pkg.SparseAttentionMode.TRISHAPE), ("num_last_dense_tokens_in_prefill", 100),
                          ("num_retained_start_tokens_in_cache", 128), ("num_retained_recent_tokens_in_cache", 1920),
                          ("xattention_threshold", 0.8), ("xattention_block_size", 64), ("xattention_stride", 8)):
        assert getattr(sp, name) == default
    sc.use_sparse_attention = True
    assert "sparseAttentionMode: TRISHAPE" in sc.to_string() and "xattention_stride: 8" in sc.to_string()


def test_pipeline_metrics_keep_reference_names_and_bookkeeping(pkg):
    # fields: include/openvino/genai/continuous_batching_pipeline.hpp:33-75; Python names:
    # src/python/py_continuous_batching_pipeline.cpp:461-467
    m = pkg.PipelineMetrics()
    for name in ("requests", "scheduled_requests", "cache_usage", "avg_cache_usage", "cache_size_in_bytes",
                 "kv_cache_size_in_bytes", "max_cache_usage", "inference_duration", "sampling_duration"):
        assert getattr(m, name) == 0
    m.cache_size_in_bytes = 7
    assert m.kv_cache_size_in_bytes == 7
    # BlockAllocator::get_used_percentage (block_manager.hpp:588-592) in float32: 2 layers x 10 blocks, 3 + 4 free
    assert pkg.used_percentage([3, 4], 10) == float(np.float32(13) / np.float32(20) * np.float32(100)) == 65.0
    assert pkg.used_percentage([10, 10], 10) == 0.0 and pkg.used_percentage([0], 3) == 100.0
    t = pkg.PipelineMetricsTracker()
    usages = []
    for step in range(1200):                    # pipeline_impl.cpp:394-398 with the 1000-step window of :779-789
        free = [step % 7, (3 * step) % 11]
        usages.append(t.register_step(free, 16, requests=5, scheduled_requests=3, cache_size_in_bytes=1 << 20))
        got = t.get_metrics()
        assert got.cache_usage == usages[-1] and got.max_cache_usage == max(usages)
        assert got.avg_cache_usage == float(np.float32(sum(usages[-1000:]) / len(usages[-1000:])))
    assert (got.requests, got.scheduled_requests, got.cache_size_in_bytes) == (5, 3, 1 << 20)
    waited = []
    with t.time_forward(lambda: waited.append(1)):
        pass
    assert waited == [1] and 0.0 < t.get_metrics().inference_duration < 1e6
    t.reset_cache_usage_statistics()            # :791-795: maximum and average start over, the last usage stays
    got = t.get_metrics()
    assert (got.max_cache_usage, got.avg_cache_usage) == (0.0, 0.0) and got.cache_usage == usages[-1]
    t.register_step([8], 16)
    assert t.get_metrics().avg_cache_usage == 50.0


def test_xattention_threshold_schedule(pkg):
    """Scheduler::_schedule_xattention_threshold (scheduler.hpp:922-940): library against the checker's restatement."""
    from oracle import oracle as O
    cfg = pkg.SparseAttentionConfig(mode=pkg.SparseAttentionMode.XATTENTION, xattention_threshold=0.9,
                                    num_last_dense_tokens_in_prefill=100)
    assert pkg.schedule_xattention_threshold(pkg.SparseAttentionConfig(), 1000, 0, 256, False) == 0.0  # TRISHAPE mode
    assert pkg.schedule_xattention_threshold(cfg, 1000, 0, 256, False, use_sparse_attention=False) == 0.0
    import itertools
    for prompt, processed, scheduled, gen in itertools.product((1000, 130), (0, 512, 899, 900, 1000), (1, 100, 388, 389, 488),
                                                               (False, True)):
        want = O.xattention_threshold(np.float32(0.9), 100, prompt, processed, scheduled, gen)
        assert pkg.schedule_xattention_threshold(cfg, prompt, processed, scheduled, gen) == want


@pytest.mark.parametrize("c", K.KATS["invalid_config"]["config_cases"])
def test_invalid_eviction_config_throws(pkg, c):
    with pytest.raises(ValueError):
        pkg.CacheEvictionConfig(c[0], c[1], c[2], pkg.AggregationMode.NORM_SUM, False, 8)


def test_create_without_gpu_fails_cleanly(pkg):
    torch = pytest.importorskip("torch")
    if torch.cuda.is_available():
        pytest.skip("a GPU is present")
    with pytest.raises(pkg.PaError):
        pkg.PagedAttention(8, 2, 128)


def test_package_raises_when_the_hip_library_is_missing():
    """No CPU fallback: with the library absent the first use of the package raises and names the file."""
    import os
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    code = ("import __graft_entry__ as g\n"
            "try:\n"
            "    pkg = g.load_package()\n"
            "    pkg.pack_step([3], [0], [0], [1], [1], 32)\n"
            "except ImportError as e:\n"
            "    print('RAISED', e)\n"
            "else:\n"
            "    print('NO ERROR')\n")
    env = dict(os.environ, PA_AMD_LIBRARY="/nonexistent/libpa_amd.so")
    r = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, cwd=root, env=env, timeout=300)
    assert "RAISED" in r.stdout and "/nonexistent/libpa_amd.so" in r.stdout and "no CPU fallback" in r.stdout, r.stdout + r.stderr


def test_the_product_never_refers_to_the_checker():
    """The CPU checker is test infrastructure: nothing under the package or the header names it, the benchmark only
    inside its CPU-baseline leg, the entry module only to build it and (through the tests' harness) in smoke()."""
    import os
    import re
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    for base in ("openvino.genai_amd", "include"):
        for d, _, files in os.walk(os.path.join(root, base)):
            for f in files:
                if f.endswith((".py", ".hip", ".h", ".cpp", "Makefile")):
                    text = open(os.path.join(d, f), encoding="utf-8").read()
                    assert "oracle" not in text and "_work/" not in text, os.path.join(d, f)
    bench = open(os.path.join(root, "bench.py"), encoding="utf-8").read()
    uses = [m.start() for m in re.finditer(r"\boracle\b", bench)]
    leg = bench.index("def cpu_baseline(")
    leg_end = bench.index("\ndef ", leg + 1)
    assert uses and all(leg < u < leg_end for u in uses)
    assert "_work/" not in bench
