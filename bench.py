"""Benchmark of the PagedAttention decode path on one MI355X.

A step is one layer's PagedAttention call (KV append + u8 quantisation of the new tokens, split-K decode attention,
per-token score emission) over the headline workload: Llama-3-8B shape (32 query heads, 8 KV heads, head size 128,
block 32), u8 KV cache, 64 sequences at 4096 tokens of context, block tables = random permutation over a 2x pool.
All tensors are resident in HBM before the timed region; contents are synthetic (seeded normal + 1 % outliers at
+-8, quantised into the cache by the library's own append kernel).

Prints one JSON line.  `value` = algorithmic bytes of a step / step time; `roofline` prices the dominant kernel
(the decode attention kernel, timed alone with HIP events on its stream) against the 8 TB/s HBM peak;
`cpu_baseline` times the CPU checker's restatement of the same call on the host cores.
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0
NUM_LAYERS_FOR_TOKS = 32  # Llama-3-8B depth: tok/s = batch / (32 * t_layer), attention only

# HBM bytes per launch of the dominant kernel: not measured by this script but read off rocprofv3 --pmc FETCH_SIZE /
# WRITE_SIZE runs of it, scaled by the readings of a plain 1 GiB copy; the summary file holds commands and readings.
# (a workload without a reading of the kernel as it stands is not listed: `traffic` is then null)
MEASURED_TRAFFIC = {
    "llama3_8b_decode_u8_b64_ctx4096": (581.0e6, "profiles/pa_decode_u8_kernel__llama3_8b_decode_u8_b64_ctx4096.md"),
    "llama3_8b_eviction_u8_b256_ctx8192": (4622.7e6, "profiles/pa_decode_u8_kernel__llama3_8b_eviction_u8_b256_ctx8192.md"),
    "long_context_decode_u8_b8_ctx32768": (594.4e6, "profiles/pa_decode_u8_kernel__long_context_decode_u8_b8_ctx32768.md"),
    "qwen25_7b_mixed_bf16": (218.8e6, "profiles/pa_prefill16_kernel__qwen25_7b_mixed_bf16.md"),
    "phi3_mini_decode_u8_b64_ctx4096": (1777.6e6, "profiles/pa_decode_kernels__head_sizes_96_256_decode_b64_ctx4096.md"),
    "gemma2_9b_decode_u8_b64_ctx4096": (1122.3e6, "profiles/pa_decode_kernels__head_sizes_96_256_decode_b64_ctx4096.md"),
}


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--config", type=int, default=2, help="workload (2 = headline; 1, 4, 5, other head sizes 6, 7 and larger prefill steps 8, 9 for diagnostics)")
    ap.add_argument("--batch", type=int, default=None)
    ap.add_argument("--sliding-window", type=int, default=None)
    ap.add_argument("--new-tokens", type=int, default=None,
                    help="decode workloads: every sequence schedules this many tokens (a speculative-decoding validation step)")
    ap.add_argument("--block-size", type=int, choices=[16, 32], default=None,
                    help="KV block size of the workload (default: the configuration's, 32)")
    ap.add_argument("--kv-dtype", choices=["u8", "f16", "bf16"], default=None,
                    help="diagnostics: run the workload's shape over another cache type")
    ap.add_argument("--cache-tensors", choices=["manager", "torch"], default="manager",
                    help="who allocates key_cache / value_cache: the library's cache manager (as under the pipeline) or torch")
    ap.add_argument("--no-scores", action="store_true")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--cpu-seconds", type=float, default=12.0, help="wall-clock budget of the CPU baseline")
    ap.add_argument("--settle-steps", type=int, default=2000,
                    help="untimed steps run before the warmup so that the GPU's clocks have settled when the timed "
                         "steps start (a few thousand steps are a few tenths of a second); reported in `config`")
    ap.add_argument("--layers", type=int, default=32,
                    help="decoder layers of the eviction leg of --config 4 (score registration and eviction run over "
                         "every layer of every sequence in one call)")
    ap.add_argument("--evict-modes", default="norm_sum,kvcrush,adaptive_rkv",
                    help="eviction legs of --config 4 beside NORM_SUM: kvcrush, adaptive_rkv (comma separated); none = no eviction leg")
    ap.add_argument("--diversity", type=int, default=0, metavar="TOKENS",
                    help="adds a leg: ADAPTIVE_RKV block diversity over an evictable area of this many tokens (a "
                         "multiple of 32) of every sequence, behind a start area of 32 tokens")
    ap.add_argument("--xattention", type=float, default=0.0, metavar="THRESHOLD",
                    help="adds a leg: block-sparse prefill with this threshold against dense prefill (4 x 512-token "
                         "chunks, Qwen2.5-7B shape, bf16 cache)")
    ap.add_argument("--append", type=int, default=0, metavar="TOKENS",
                    help="also time pa_kv_append for one sequence of TOKENS new tokens (the workload's heads and cache type)")
    ap.add_argument("--rotate", action="store_true",
                    help="adds a leg: cache rotation (the re-rotation of K rows behind evicted blocks) over every "
                         "block of the workload's sequences, one layer")
    ap.add_argument("--kv-cache-leg", action="store_true",
                    help="adds a leg: copy-on-write of 256 blocks x 32 layers and growth of the cache tensors")
    ap.add_argument("--pool-factor", type=float, default=2.0,
                    help="size of the block pool the tables are drawn from, as a multiple of the blocks in use")
    ap.add_argument("--flush-mb", type=int, default=1024,
                    help="size of the scratch buffer read before every launch of the second, cold kernel-only "
                         "measurement (displaces what the previous launch left in L2 / Infinity Cache); 0 = skip it")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run a plain 1 GiB device copy (reference reading for rocprofv3 FETCH_SIZE / WRITE_SIZE)")
    return ap.parse_args()


class _DeviceBytes:
    """A run of device memory owned by someone else, presented through the array interface torch reads."""

    def __init__(self, ptr, nbytes):
        self.__cuda_array_interface__ = {"shape": (nbytes,), "typestr": "|u1", "data": (int(ptr), False), "version": 2}


def cache_view(torch, ptr, shape, dev):
    """A uint8 tensor over a cache tensor of the library's cache manager (no copy; the manager keeps the memory)."""
    t = torch.as_tensor(_DeviceBytes(ptr, int(np.prod(shape))), device=dev).view(*shape)
    assert t.data_ptr() == int(ptr)
    return t


def fill_cache(torch, op, spec, kc, vc, dev, gen):
    """Fills the past of every sequence through the library's append kernel, a few sequences at a time."""
    B, Hkv, D = spec["B"], spec["Hkv"], spec["D"]
    dt = torch.float16 if spec["q_dtype"] == "f16" else torch.bfloat16
    past = spec["past_lens"].astype(np.int64)
    bib = spec["block_indices_begins"]
    group = max(1, int(2 ** 27 // max(1, int(past.max()) * Hkv * D)))
    for b0 in range(0, B, group):
        b1 = min(B, b0 + group)
        p = past[b0:b1]
        if p.sum() == 0:
            continue
        sb = np.concatenate([[0], np.cumsum(p)]).astype(np.int32)
        T = int(sb[-1])
        k = torch.randn(T, Hkv * D, generator=gen, device=dev, dtype=torch.float32)
        v = torch.randn(T, Hkv * D, generator=gen, device=dev, dtype=torch.float32)
        for x in (k, v):  # 1 % outliers at +-8
            m = torch.rand(x.shape, generator=gen, device=dev) < 0.01
            s = torch.where(torch.rand(x.shape, generator=gen, device=dev) < 0.5, 8.0, -8.0)
            x[m] = s[m]
        keep = p > 0
        op.step_begin(np.zeros(int(keep.sum()), np.int32), np.concatenate([[0], np.cumsum(p[keep])]).astype(np.int32),
                      np.concatenate([[0], np.cumsum((bib[b0 + 1:b1 + 1] - bib[b0:b1])[keep])]).astype(np.int32))
        ids = np.concatenate([spec["block_indices"][bib[b0 + i]:bib[b0 + i + 1]] for i in range(b1 - b0) if keep[i]])
        op.set_block_indices(ids, spec["num_blocks"])
        op.kv_append(k.to(dt), v.to(dt), kc, vc)
        op.synchronize()


def cpu_baseline(spec, seconds, with_scores, q, kc, vc):
    """Times the CPU checker on the inputs of the GPU leg: the same query rows, caches (as the library's append
    kernel quantised them) and block table, copied to the host."""
    from oracle import oracle as O
    threads = min(os.cpu_count() or 1, 16)
    Hq, Hkv, D, bs = spec["Hq"], spec["Hkv"], spec["D"], spec["bs"]
    dt = {"f16": O.DT_F16, "bf16": O.DT_BF16, "u8": O.DT_U8}
    table = spec["block_indices"]

    def timed(n_threads, budget):
        times = []
        t_start = time.perf_counter()
        while not times or time.perf_counter() - t_start < budget:
            t0 = time.perf_counter()
            O.paged_attention(q, dt[spec["q_dtype"]], kc, vc, dt[spec["kv_dtype"]], spec["past_lens"],
                              spec["subsequence_begins"], table, spec["block_indices_begins"], Hq, Hkv, D, bs,
                              spec["scale"], spec["sliding_window"], None, with_scores, n_threads)
            times.append(time.perf_counter() - t0)
        return float(np.mean(times)), len(times)

    t_all, n_all = timed(threads, seconds)
    t_one, _ = timed(1, min(2.0, seconds / 4))  # one thread alongside: a pass or a few
    return t_all, n_all, threads, t_one


def cpu_model():
    """What /proc/cpuinfo says of the first CPU: model name, vendor, family / model / stepping, clock."""
    want = ("model name", "vendor_id", "cpu family", "model", "stepping", "cpu MHz")
    got = {}
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if ":" not in line:
                    if got:
                        break
                    continue
                key, val = (x.strip() for x in line.split(":", 1))
                if key in want and key not in got:
                    got[key] = val
    except OSError:
        return "unknown"
    return "%s (%s, family %s model %s stepping %s, %s MHz)" % (
        got.get("model name", "unknown"), got.get("vendor_id", "?"), got.get("cpu family", "?"), got.get("model", "?"),
        got.get("stepping", "?"), got.get("cpu MHz", "?"))


def eviction_leg(torch, pkg, op, spec, q, kc, vc, out, scores, dev, layers, mode="norm_sum"):
    """Score accumulation + eviction on the device for the scoring workload, every layer of every sequence in one
    call (the layers share one scores tensor here): the first registration sees the whole 8193-token context and
    evicts down to max_cache_size; the steady state registers a 1024-token cache's scores plus one block of new
    tokens and evicts one block per sequence and layer in every timed step (the step that comes up once per
    block_size generated tokens; the steps between register only).
    Times are host wall clock around the C-ABI calls (upload of the per-pair entries, launches, read-back of the
    evicted block lists included), buffers preallocated.
    mode: "norm_sum"; "kvcrush" (NORM_SUM with a KVCrush budget of 8 blocks, MEAN anchor: some of the chosen blocks
    stay as representatives); "adaptive_rkv" (a block diversity matrix is registered before every eviction, as the
    pipeline does with the op's `adaptive_rkv_diversity.<L>` output -- synthetic values here, one tensor for all
    layers; its first eviction runs over 2 layers, the diversity of 8000 evictable tokens being 8 MB per pair)."""
    import ctypes as C
    from openvino_genai_amd import _lib as L
    B, bs = spec["B"], spec["bs"]
    rkv = mode == "adaptive_rkv"
    agg = pkg.AggregationMode.ADAPTIVE_RKV if rkv else pkg.AggregationMode.NORM_SUM
    crush = pkg.KVCrushConfig(8, pkg.KVCrushAnchorPointMode.MEAN) if mode == "kvcrush" else None
    cfg = pkg.CacheEvictionConfig(32, 128, 1024, agg, False, 0, crush)
    cfg_every = pkg.CacheEvictionConfig(32, 128, 1024, agg, False, 0, pkg.KVCrushConfig(1, pkg.KVCrushAnchorPointMode.MEAN))
    lib = L.lib()
    slots = np.arange(B, dtype=np.int32)
    p32 = lambda a: a.ctypes.data_as(C.POINTER(C.c_int32))
    p64 = lambda a: a.ctypes.data_as(C.POINTER(C.c_int64))
    start = 32

    def make(n_layers, score_tensor=None, config=cfg):
        ev = pkg.Evictor(config, bs, n_layers, 7, max_sequences=B, max_tracked_tokens=8448, device=0,
                         stream=torch.cuda.current_stream(dev))
        ptrs = (C.c_void_p * n_layers)(*[C.c_void_p((scores if score_tensor is None else score_tensor).data_ptr())] * n_layers)
        counts = np.zeros(B * n_layers, np.int32)
        blocks = np.empty(B * n_layers * 256, np.int32)
        blocks.fill(0)  # (touched here: the first write into fresh pages is not the library's time)

        def register(offsets):
            L.check(lib.pa_evictor_register_scores(ev._h, B, p32(slots), ptrs, p64(offsets), None), lib.pa_evictor_last_error, ev._h)

        pool = {}

        def diversity():  # [n / bs, n] floats per sequence for the eviction that is due, the same tensor for every layer
            rb_, re_ = ev.get_evictable_block_range(0, 0)
            n_evictable = (re_ - rb_) * bs
            per = (n_evictable // bs) * n_evictable
            if pool.get("n", 0) < B * per:
                pool["t"] = -torch.rand(B * per, device=dev, dtype=torch.float32)
                pool["n"] = B * per
            off = (np.arange(B + 1, dtype=np.int64) * per)
            dp = (C.c_void_p * n_layers)(*[C.c_void_p(pool["t"].data_ptr())] * n_layers)
            return pool["t"], off, dp

        def register_diversity(d):
            L.check(lib.pa_evictor_register_block_diversity(ev._h, B, p32(slots), d[2], p64(d[1])), lib.pa_evictor_last_error, ev._h)

        def evict():
            L.check(lib.pa_evictor_evict(ev._h, B, p32(slots), p32(counts), p32(blocks), 256), lib.pa_evictor_last_error, ev._h)

        return ev, register, diversity, register_diversity, evict, counts

    kv = spec["past_lens"].astype(np.int64) + 1
    offsets = np.concatenate([[0], np.cumsum(kv)]).astype(np.int64)
    op.attention(q, kc, vc, out, scores)
    # the first launch of a kernel also loads its code: a throw-away evictor takes that
    warm = pkg.Evictor(cfg, bs, 1, 7, max_sequences=1, max_tracked_tokens=8448, device=0, stream=torch.cuda.current_stream(dev))
    warm.register_new_token_scores([0], [scores.data_ptr()], [0, 2000], None)
    if rkv:
        n0 = (2000 - start - 128) // bs * bs
        wd = -torch.rand((n0 // bs) * n0, device=dev, dtype=torch.float32)
        warm.register_block_diversity([0], [wd.data_ptr()], [0, wd.numel()])
    warm.evict_logical_blocks([0], max_blocks_per_entry=256)
    del warm
    torch.cuda.synchronize(dev)
    # ---- first registration + eviction over the whole context
    first_layers = min(layers, 2) if rkv else layers
    ev, register, diversity, register_diversity, evict, counts = make(first_layers)
    t0 = time.perf_counter()
    register(offsets)
    torch.cuda.synchronize(dev)
    t1 = time.perf_counter()
    t_div = 0.0
    d = None
    if rkv:
        d = diversity()
        torch.cuda.synchronize(dev)
        a = time.perf_counter()
        register_diversity(d)
        torch.cuda.synchronize(dev)
        t_div = time.perf_counter() - a
        t1 = time.perf_counter()
    evict()
    torch.cuda.synchronize(dev)
    t2 = time.perf_counter()
    first_counts = counts.copy()
    tracked = int((kv - 32).sum()) * first_layers
    d = None
    del ev
    t_distinct = None
    if mode == "kvcrush":
        # KVCrush marks the better half of the tokens; where that half ends inside a run of equal scores the choice
        # is the host sorting routine's and the library walks that entry's scores on the host (threads).  This
        # synthetic workload's scores underflow to exactly 0 for most of the context; uniform random scores still tie,
        # because max pooling (window 7, the pipeline's) repeats a local maximum over its neighbours.  With a budget
        # of 8 the steady state's one block per step is below the budget and nothing is thinned; `_budget_1` is the
        # steady state where every eviction is.
        distinct = torch.rand(scores.numel(), device=dev, dtype=torch.float32)
        ev, register, diversity, register_diversity, evict, counts = make(first_layers, distinct)
        register(offsets)
        torch.cuda.synchronize(dev)
        a = time.perf_counter()
        evict()
        t_distinct = time.perf_counter() - a
        del ev, distinct
    # ---- steady state: a block of new tokens per sequence on a 1024-token cache (scores of the capped context)
    def steady(config):
        ev, register, diversity, register_diversity, evict, counts = make(layers, None, config)
        kv2 = np.full(B, 1024, np.int64)
        register(np.concatenate([[0], np.cumsum(kv2)]).astype(np.int64))  # (brings the slots to the capped length, untimed)
        torch.cuda.synchronize(dev)
        kv2 = kv2 + 33
        reg, evi, both, most = [], [], [], []
        for _ in range(12):
            off2 = np.concatenate([[0], np.cumsum(kv2)]).astype(np.int64)
            a = time.perf_counter()
            register(off2)
            if rkv:
                register_diversity(diversity())
            b_ = time.perf_counter()   # (the registration is left in flight: the eviction follows on the same stream)
            evict()
            c_ = time.perf_counter()
            reg.append(b_ - a)
            evi.append(c_ - b_)
            both.append(c_ - a)
            most.append(int(counts.max()))
            # what stays: a retained representative makes the next eviction take two blocks
            kv2 = kv2 - counts.reshape(B, layers)[:, 0].astype(np.int64) * bs + bs  # a block of new tokens per step
        torch.cuda.synchronize(dev)
        return reg, evi, both, most

    reg, evi, both, steady_counts = steady(cfg)
    every = steady(cfg_every) if mode == "kvcrush" else None
    return {"mode": mode, "layers": layers, "sequences": B, "first_eviction_layers": first_layers,
            "first_register_ms": round((t1 - t0 - t_div) * 1e3, 3), "first_evict_ms": round((t2 - t1) * 1e3, 3),
            "first_register_diversity_ms": round(t_div * 1e3, 3) if rkv else None,
            "first_evict_ms_uniform_random_scores": round(t_distinct * 1e3, 3) if t_distinct is not None else None,
            "steady_evict_call_ms_budget_1": round(float(np.median(every[1])) * 1e3, 3) if every else None,
            "steady_register_plus_evict_ms_budget_1": round(float(np.median(every[2])) * 1e3, 3) if every else None,
            "first_register_GBps": round(tracked * 20 / (t1 - t0 - t_div) / 1e9, 1),
            "blocks_evicted_per_sequence_and_layer_first": [int(first_counts.min()), int(first_counts.max())],
            "blocks_evicted_per_entry_steady_max": steady_counts,
            "steady_register_call_ms": round(float(np.median(reg)) * 1e3, 3),
            "steady_evict_call_ms": round(float(np.median(evi)) * 1e3, 3),
            "steady_register_plus_evict_ms": round(float(np.median(both)) * 1e3, 3),
            "note": "host wall clock per C-ABI call, %d sequences x %d layers per call; the steady-state pair is timed "
                    "as one (register returns with its kernel in flight, evict returns with the block lists on the "
                    "host; ADAPTIVE_RKV: the registration of the diversity matrices counts as registration); "
                    "first_register_GBps prices 20 bytes per tracked token (4 read, 16 written)" % (B, layers)}


def kv_cache_leg(torch, pkg, dev, layers=32, blocks=256):
    """Block-table maintenance on the device: copy-on-write of `blocks` blocks in every layer's K and V tensor (one
    call), and growth of the cache from N to 2N blocks (Llama-3-8B shape, u8).  Host wall clock around the
    synchronous C-ABI calls."""
    mgr = pkg.KVCacheManager(layers, 8, 128, 32, "u8")
    bb = mgr.get_block_size_in_bytes()
    n = 4 * blocks
    t0 = time.perf_counter()
    mgr.allocate_cache_if_needed(n)
    t1 = time.perf_counter()
    first_ptr = mgr.get_key_cache(0)
    times = []
    for r in range(6):
        copy_map = {int(i): [2 * blocks + (int(i) + r) % blocks] for i in range(blocks)}
        a = time.perf_counter()
        mgr.copy_blocks(copy_map)
        times.append(time.perf_counter() - a)
    t2 = time.perf_counter()
    mgr.allocate_cache_if_needed(2 * n)
    t3 = time.perf_counter()
    assert mgr.get_key_cache(0) == first_ptr
    ms = float(np.median(times[1:])) * 1e3
    moved = 2.0 * blocks * bb  # read + written
    return {"layers": layers, "blocks_copied": blocks, "copy_blocks_ms": round(ms, 4),
            "copy_blocks_GBps": round(moved / (ms * 1e-3) / 1e9, 1),
            "roofline": {"bound": "hbm", "kernel": "kv_copy_blocks_kernel", "achieved": round(moved / (ms * 1e-3) / 1e9, 1),
                         "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": round(moved / (ms * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4)},
            "first_allocation_ms": round((t1 - t0) * 1e3, 3), "growth_to_twice_ms": round((t3 - t2) * 1e3, 3),
            "cache_bytes_after_growth": 2 * n * bb,
            "note": "copy: one upload of the pair list, one launch over (pair, layer, K|V), one stream wait; bytes = "
                    "blocks x block bytes over all layers, read + written.  Growth maps new memory behind the tensors' "
                    "fixed base addresses and clears it; nothing is copied"}


def diversity_leg(torch, op, spec, kc, dev, ev, reps=20):
    """Block diversity of an `ev`-token evictable area of every sequence (one layer), timed with events on the
    launch stream around `reps` calls; the figure includes the call's own upload and launches."""
    B, Hkv, D, bs = spec["B"], spec["Hkv"], spec["D"], spec["bs"]
    ev = min(ev, (int(spec["past_lens"].min()) + 1 - 32) // bs * bs)
    sizes = [ev] * B
    out = torch.zeros(B * (ev // bs) * ev, dtype=torch.float32, device=dev)
    for _ in range(3):
        op.adaptive_rkv_diversity(kc, 32, sizes, out)
    torch.cuda.synchronize(dev)
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(reps):
        op.adaptive_rkv_diversity(kc, 32, sizes, out)
    e1.record()
    torch.cuda.synchronize(dev)
    ms = e0.elapsed_time(e1) / reps
    flops = 2.0 * D * ev * ev * Hkv * B
    peak = 2500.0
    return {"evictable_tokens": ev, "sequences": B, "ms_per_call": round(ms, 4), "flops": flops,
            "roofline": {"bound": "mfma", "kernel": "rkv_diversity_kernel", "achieved": round(flops / (ms * 1e-3) / 1e12, 2),
                         "peak": peak, "unit": "TFLOP/s", "frac": round(flops / (ms * 1e-3) / 1e12 / peak, 4)},
            "note": "2 * D flops per (token pair, kv head); wall time of the whole call (four kernels, one upload)"}


def rotation_leg(torch, pkg, op, spec, kc, dev, reps=10):
    """Cache rotation of every block of the workload's sequences (one layer, one delta per block): wall time of
    the whole call (argument checks, the block list and deltas copied to pinned staging and queued, one kernel),
    events on the launch stream.  Rotates a copy of the K cache, in place."""
    Hkv, D, bs = spec["Hkv"], spec["D"], spec["bs"]
    blocks = np.ascontiguousarray(spec["block_indices"], np.int32)
    rng = np.random.default_rng(77)
    max_blocks = 512
    deltas = rng.integers(1, max_blocks, size=(len(blocks), 1)).astype(np.int32)
    op.set_rotation_trig_lut(pkg.rotation_trig_lut(bs, max_blocks, D))
    work = kc.clone()
    for _ in range(2):
        op.rotate_cache(work, blocks, deltas)
    torch.cuda.synchronize(dev)
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(reps):
        op.rotate_cache(work, blocks, deltas)
    e1.record()
    torch.cuda.synchronize(dev)
    ms = e0.elapsed_time(e1) / reps
    row = D + 8 if spec["kv_dtype"] == "u8" else 2 * D
    nbytes = 2.0 * len(blocks) * Hkv * bs * row
    return {"blocks": int(len(blocks)), "ms_per_call": round(ms, 4), "bytes": nbytes,
            "roofline": {"bound": "hbm", "kernel": "pa_rotate_rows_kernel", "achieved": round(nbytes / (ms * 1e-3) / 1e9, 1),
                         "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": round(nbytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4)},
            "note": "every K row read and written once; wall time of the whole call"}


def append_leg(torch, pkg, spec, dev, tokens, reps=20):
    """KV append at prefill scale: one sequence of ``tokens`` new tokens from scratch, the workload's heads and cache
    type; the step's K and V rows read once, their cache rows written once.  Events around ``reps`` calls of
    pa_kv_append on the launch stream."""
    Hq, Hkv, D, bs = spec["Hq"], spec["Hkv"], spec["D"], spec["bs"]
    stream = torch.cuda.current_stream(dev)
    op = pkg.PagedAttention(Hq, Hkv, D, bs, spec["q_dtype"], spec["kv_dtype"], num_layers=1, device=0, stream=stream)
    nblk = (tokens + bs - 1) // bs
    rb = pkg.row_bytes(D, spec["kv_dtype"])
    kc = torch.zeros(nblk, Hkv, bs, rb, dtype=torch.uint8, device=dev)
    vc = torch.zeros_like(kc)
    dt = torch.float16 if spec["q_dtype"] == "f16" else torch.bfloat16
    gen = torch.Generator(device=dev).manual_seed(4242)
    k = torch.randn(tokens, Hkv * D, generator=gen, device=dev, dtype=torch.float32).to(dt)
    v = torch.randn(tokens, Hkv * D, generator=gen, device=dev, dtype=torch.float32).to(dt)
    op.step_begin(np.zeros(1, np.int32), np.array([0, tokens], np.int32), np.array([0, nblk], np.int32), tokens)
    op.set_block_indices(np.random.default_rng(5).permutation(nblk).astype(np.int32), nblk)
    for _ in range(3):
        op.kv_append(k, v, kc, vc)
    torch.cuda.synchronize(dev)
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(reps):
        op.kv_append(k, v, kc, vc)
    e1.record()
    torch.cuda.synchronize(dev)
    ms = e0.elapsed_time(e1) / reps
    nbytes = 2.0 * tokens * Hkv * (2 * D + rb)
    return {"tokens": tokens, "ms_per_call": round(ms, 4), "bytes": nbytes,
            "roofline": {"bound": "hbm", "kernel": "kv_append_tokens_kernel" if tokens >= 8192 else "kv_append_kernel",
                         "achieved": round(nbytes / (ms * 1e-3) / 1e9, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                         "frac": round(nbytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4)},
            "note": "K and V rows of the step read once, their cache rows written once"}


def xattention_leg(torch, pkg, dev, threshold, kv_dtype="bf16", reps=20):
    """Block-sparse prefill (XAttention, block 64, stride 8) against dense prefill on the prefill part of the mixed
    workload: four 512-token chunks at past 0 / 2048 / 4096 / 8192, Qwen2.5-7B shape, bf16 cache (u8 with --kv-dtype u8).  Plain N(0,1) data
    attends almost uniformly, which no threshold can prune, so the keys here have structure of the kind trained
    models show: the first 64 tokens and 4 % of the other 64-token blocks of every sequence ("sinks" and
    "retrieval" blocks) lie along a direction the queries of their kv head share, and draw most of the attention.
    Times are per call (events on the launch stream, all kernels of the call)."""
    Hq, Hkv, D, bs = 28, 4, 128, 32
    past = np.array([0, 2048, 4096, 8192], np.int32)
    new = np.full(4, 512, np.int32)
    sb = np.concatenate([[0], np.cumsum(new)]).astype(np.int32)
    nblk = (past + new + bs - 1) // bs
    bib = np.concatenate([[0], np.cumsum(nblk)]).astype(np.int32)
    pool = int(bib[-1]) * 2
    rng = np.random.default_rng(1003)
    table = rng.permutation(pool)[:bib[-1]].astype(np.int32)
    gen = torch.Generator(device=dev).manual_seed(1003)
    op = pkg.PagedAttention(Hq, Hkv, D, bs, "bf16", kv_dtype, num_layers=1, device=0, stream=torch.cuda.current_stream(dev))
    u = torch.randn(Hkv, D, generator=gen, device=dev)
    # the whole contexts as one prefill through the library's own append (which also quantises u8 caches)
    kv_len = (past + new).astype(np.int32)
    ctx_sb = np.concatenate([[0], np.cumsum(kv_len)]).astype(np.int32)
    kf = torch.randn(int(ctx_sb[-1]), Hkv, D, generator=gen, device=dev)
    for b in range(4):
        n64 = int(kv_len[b]) // 64
        heavy = [0] + [int(x) for x in np.nonzero(rng.random(n64) < 0.04)[0] if x > 0]
        for h64 in heavy:
            kf[ctx_sb[b] + 64 * h64: ctx_sb[b] + 64 * h64 + 64] += 0.85 * u[None]
    vf = torch.randn(int(ctx_sb[-1]), Hkv * D, generator=gen, device=dev).to(torch.bfloat16)
    rb = pkg.row_bytes(D, kv_dtype)
    kc = torch.zeros(pool, Hkv, bs, rb, dtype=torch.uint8, device=dev)
    vc = torch.zeros_like(kc)
    op.step_begin(np.zeros(4, np.int32), ctx_sb, bib, int(kv_len.max()))
    op.set_block_indices(table, pool)
    op.kv_append(kf.reshape(-1, Hkv * D).to(torch.bfloat16), vf, kc, vc)
    op.synchronize()
    del kf, vf
    T = int(sb[-1])
    q = (torch.randn(T, Hq, D, generator=gen, device=dev) + 0.85 * u.repeat_interleave(Hq // Hkv, 0)[None]) \
        .reshape(T, Hq * D).to(torch.bfloat16)
    out = torch.zeros_like(q)

    def timed(thr):
        op.step_begin(past, sb, bib, int((past + new).max()), None, 0, 0.0)
        op.set_block_indices(table, pool)
        op.set_xattention(thr, 64, 8)
        for _ in range(3):
            op.attention(q, kc, vc, out)
        torch.cuda.synchronize(dev)
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(reps):
            op.attention(q, kc, vc, out)
        e1.record()
        torch.cuda.synchronize(dev)
        return e0.elapsed_time(e1) / reps, out.float().clone()

    dense_ms, dense_out = timed(None)
    sparse_ms, sparse_out = timed(np.full(4, threshold, np.float32))
    kept = pairs = 0
    for b in range(4):
        r = op.xattention_retained(b)
        qb0, nqb, nkb = op.xattention_shape(b)
        vis = np.tril(np.ones((nqb, nkb), np.int64), k=qb0)
        kept += int((r * vis).sum())
        pairs += int(vis.sum()) * Hq
    est_flops = 2.0 * D / 8 * Hq * sum(float(n) * (p + (n + 1) / 2) for p, n in zip(past, new))
    diff = (sparse_out - dense_out).abs()
    return {"threshold": threshold, "kv_dtype": kv_dtype, "xattention_block_size": 64, "xattention_stride": 8,
            "dense_ms": round(dense_ms, 4), "sparse_ms": round(sparse_ms, 4),
            "kept_block_pairs": round(kept / pairs, 4), "estimate_flops": est_flops,
            "sparse_vs_dense_output": {"max_abs": round(float(diff.max()), 4), "mean_abs": round(float(diff.mean()), 5),
                                       "dense_mean_abs": round(float(dense_out.abs().mean()), 5)},
            "note": "sparse_ms includes the estimate (strided logits; statistics, block sums and selection; the work "
                    "items' block lists) and the block-masked matrix kernel; per-kernel times are in the rocprofv3 "
                    "summary.  The output difference is what the approximation costs on this data, not an error."}


def main():
    args = parse()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU only; --gpus %d is not supported (no collective, no sharding "
              "code is part of it)." % args.gpus, file=sys.stderr)
        sys.exit(2)
    import torch
    import __graft_entry__ as entry
    pkg = entry.load_package()
    wl = __import__("openvino_genai_amd.workloads", fromlist=["x"])
    assert torch.cuda.is_available(), "bench.py needs the GPU"
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)

    spec = wl.make_spec(args.config, batch=args.batch, sliding_window=args.sliding_window, pool_factor=args.pool_factor,
                        block_size=args.block_size, new_tokens=args.new_tokens)
    if args.new_tokens is not None:
        spec["name"] += "_new%d" % args.new_tokens
    if args.block_size is not None and args.block_size != 32:
        spec["name"] += "_block%d" % args.block_size
    if args.pool_factor != 2.0:
        spec["name"] += "_pool%g" % args.pool_factor
    if args.kv_dtype and args.kv_dtype != spec["kv_dtype"]:
        spec["kv_dtype"] = args.kv_dtype
        spec["name"] += "_kv_" + args.kv_dtype
        if args.kv_dtype != "u8":
            spec["q_dtype"] = args.kv_dtype  # 16-bit caches are used in the query's type
    B, Hq, Hkv, D, bs = spec["B"], spec["Hq"], spec["Hkv"], spec["D"], spec["bs"]
    with_scores = not args.no_scores
    stream = torch.cuda.current_stream(dev)
    op = pkg.PagedAttention(Hq, Hkv, D, bs, spec["q_dtype"], spec["kv_dtype"], num_layers=1, device=0, stream=stream)
    gen = torch.Generator(device=dev).manual_seed(1000 + args.config)
    rb = pkg.row_bytes(D, spec["kv_dtype"])
    # the cache tensors come from the library's cache manager, as they do under the pipeline (new blocks read as zero)
    if args.cache_tensors == "manager":
        cache = pkg.KVCacheManager(1, Hkv, D, bs, spec["kv_dtype"], device=0)
        cache.allocate_cache_if_needed(spec["num_blocks"])
        kc = cache_view(torch, cache.get_key_cache(0), (spec["num_blocks"], Hkv, bs, rb), dev)
        vc = cache_view(torch, cache.get_value_cache(0), (spec["num_blocks"], Hkv, bs, rb), dev)
    else:  # plain device allocations, for comparison
        kc = torch.zeros(spec["num_blocks"], Hkv, bs, rb, dtype=torch.uint8, device=dev)
        vc = torch.zeros_like(kc)
    fill_cache(torch, op, spec, kc, vc, dev, gen)

    dt = torch.float16 if spec["q_dtype"] == "f16" else torch.bfloat16
    T = int(spec["subsequence_begins"][-1])
    q = torch.randn(T, Hq * D, generator=gen, device=dev, dtype=torch.float32).to(dt)
    k = torch.randn(T, Hkv * D, generator=gen, device=dev, dtype=torch.float32).to(dt)
    v = torch.randn(T, Hkv * D, generator=gen, device=dev, dtype=torch.float32).to(dt)
    out = torch.zeros_like(q)
    op.step_begin(spec["past_lens"], spec["subsequence_begins"], spec["block_indices_begins"], spec["max_context_len"],
                  None, spec["sliding_window"], spec["scale"])
    op.set_block_indices(spec["block_indices"], spec["num_blocks"])
    scores = torch.zeros(op.total_scores, dtype=torch.float32, device=dev) if with_scores else None

    def step():
        op.forward(q, k, v, kc, vc, out, scores)

    def timed_steps():
        for _ in range(args.warmup):
            step()
        torch.cuda.synchronize(dev)
        t0 = time.perf_counter()
        for _ in range(args.steps):
            step()
        torch.cuda.synchronize(dev)
        return (time.perf_counter() - t0) * 1e3 / args.steps

    # The same W + K steps first as a fresh process finds the GPU (clocks not yet settled), reported beside the
    # settled figure so that the record shows how much of it is the kernel and how much the clocks.
    unsettled_ms = timed_steps() if args.settle_steps > 0 else None
    for _ in range(args.settle_steps):  # clocks settle; not part of the warmup, not timed
        step()
    torch.cuda.synchronize(dev)
    ms_per_step = timed_steps()

    # the dominant kernel alone: the library brackets it with HIP events on its launch stream
    op.set_profiling(True)
    kernel_ms, cold_ms = [], []
    for i in range(args.steps):
        op.attention(q, kc, vc, out, scores)
        kernel_ms.append(op.last_kernel_ms())
    # the same launches again, each after a read-only sweep over a scratch buffer (no dirty lines whose write-back
    # would compete with the kernel): what a launch costs when nothing of its inputs is left in the caches, as in a
    # model whose layers each have their own KV cache
    flush = torch.zeros(args.flush_mb << 18, dtype=torch.int32, device=dev) if args.flush_mb > 0 else None
    for i in range(args.steps if flush is not None else 0):
        flush.max()
        op.attention(q, kc, vc, out, scores)
        cold_ms.append(op.last_kernel_ms())
    del flush
    op.set_profiling(False)
    p10, p50, p90 = (float(x) for x in np.percentile(kernel_ms, [10, 50, 90]))
    attn_ms = p50  # the roofline figures price the median launch
    attn_mean_ms = float(np.mean(kernel_ms))

    if args.calibrate_copy:
        src = torch.empty(1 << 30, dtype=torch.uint8, device=dev).fill_(1)
        dst = torch.empty_like(src)
        for _ in range(5):
            dst.copy_(src)
        torch.cuda.synchronize(dev)

    bytes_ = wl.algorithmic_bytes(spec, with_scores)
    gbps = bytes_["total"] / (ms_per_step * 1e-3) / 1e9
    attn_gbps = bytes_["total"] / (attn_ms * 1e-3) / 1e9
    mixed = T > B  # multi-token sequences present: the MFMA kernel is the dominant one
    traffic, traffic_source = MEASURED_TRAFFIC.get(spec["name"], (None, None)) \
        if with_scores and args.batch is None and not args.kv_dtype else (None, None)
    # the matrix kernel is priced with the flops of the multi-token sequences only: the single-token sequences of a
    # mixed step run in a decode kernel (over 16-bit caches next to it on a second stream, so its launch time includes
    # what it loses to the neighbour)
    flops = wl.attention_flops(spec, multi_token_only=mixed)
    res = {
        "metric": "paged-attn decode GB/s (tok/s and % HBM peak alongside), Llama-3-8B shape, u8 KV, 1 GPU"
                  if args.config == 2 and spec["kv_dtype"] == "u8" else
                  "paged-attn GB/s of the step's algorithmic bytes, workload " + spec["name"] + " (diagnostic, not the headline)",
        "value": round(gbps, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 5), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": spec["kv_dtype"] + "/f32", "data": "synthetic",
        "config": {"workload": spec["name"], "batch": B, "context": int(spec["past_lens"].max()) + 1,
                   "heads": [Hq, Hkv, D], "block_size": bs, "scores": with_scores, "splits": op.num_splits,
                   "sliding_window": spec["sliding_window"], "clock_settle_steps": args.settle_steps,
                   "cache_tensors": "pa_kv_cache (the library's cache manager)" if args.cache_tensors == "manager" else "torch allocator"},
        "pct_hbm_peak": round(100.0 * gbps / HBM_PEAK_GBPS, 2),
        "tok_per_s": round(B / (NUM_LAYERS_FOR_TOKS * ms_per_step * 1e-3), 1),
        "algorithmic_bytes": bytes_,
        "roofline": {"bound": "mfma", "kernel": "pa_prefill16_kernel", "achieved": round(flops / (attn_ms * 1e-3) / 1e12, 2),
                     "peak": 2500.0, "unit": "TFLOP/s", "frac": round(flops / (attn_ms * 1e-3) / 1e12 / 2500.0, 4),
                     "traffic": traffic, "traffic_source": traffic_source,
                     "ms": round(attn_ms, 5), "flops": flops,
                     "hbm_GBps": round(bytes_["total"] / (attn_ms * 1e-3) / 1e9, 1)} if mixed else
                    {"bound": "hbm", "kernel": "pa_decode_u8_kernel" if spec["kv_dtype"] == "u8" else
                     ("pa_prefill16_kernel" if Hq // Hkv > 16 else "pa_decode16_kernel"), "achieved": round(attn_gbps, 1),
                     "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": round(attn_gbps / HBM_PEAK_GBPS, 4),
                     "traffic": traffic, "traffic_source": traffic_source,
                     "ms": round(attn_ms, 5)},
    }
    res["roofline"]["ms_p10_p50_p90"] = [round(p10, 5), round(p50, 5), round(p90, 5)]
    res["roofline"]["ms_mean"] = round(attn_mean_ms, 5)
    # `frac` prices the median launch; the same fraction from the mean of the launches beside it
    res["roofline"]["frac_p50"] = res["roofline"]["frac"]
    res["roofline"]["frac_mean"] = round(res["roofline"]["frac"] * attn_ms / attn_mean_ms, 4)
    if unsettled_ms is not None:
        res["unsettled"] = {"ms_per_step": round(unsettled_ms, 5),
                            "value": round(bytes_["total"] / (unsettled_ms * 1e-3) / 1e9, 1),
                            "pct_hbm_peak": round(100.0 * bytes_["total"] / (unsettled_ms * 1e-3) / 1e9 / HBM_PEAK_GBPS, 2),
                            "note": "the same %d warm-up + %d timed steps run first, before the %d settle steps: what a "
                                    "fresh process measures while the clocks still ramp" % (args.warmup, args.steps, args.settle_steps)}
    res["roofline"]["launches"] = len(kernel_ms)
    if cold_ms:
        cold = float(np.median(cold_ms))
        res["roofline"]["cold"] = {"ms": round(cold, 5), "flush_mb": args.flush_mb,
                                   "frac": round(flops / (cold * 1e-3) / 1e12 / 2500.0, 4) if mixed else
                                   round(bytes_["total"] / (cold * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4)}
    if args.xattention > 0:
        res["xattention"] = xattention_leg(torch, pkg, dev, args.xattention, "u8" if args.kv_dtype == "u8" else "bf16")
    if args.diversity > 0:
        res["adaptive_rkv_diversity"] = diversity_leg(torch, op, spec, kc, dev, args.diversity)
    if args.append > 0:
        res["kv_append"] = append_leg(torch, pkg, spec, dev, args.append)
    if args.rotate:
        res["cache_rotation"] = rotation_leg(torch, pkg, op, spec, kc, dev)
    if args.kv_cache_leg:
        res["kv_cache"] = kv_cache_leg(torch, pkg, dev)
    if args.config == 4 and args.evict_modes != "none":
        res["eviction"] = eviction_leg(torch, pkg, op, spec, q, kc, vc, out, scores, dev, args.layers)
        for mode in [m for m in args.evict_modes.split(",") if m and m != "norm_sum"]:
            res["eviction_" + mode] = eviction_leg(torch, pkg, op, spec, q, kc, vc, out, scores, dev, args.layers, mode)
    if not args.no_cpu_baseline:
        q_h = q.view(torch.int16).cpu().numpy().view(np.uint16)
        t_cpu, n_pass, threads, t_one = cpu_baseline(spec, args.cpu_seconds, with_scores, q_h, kc.cpu().numpy(), vc.cpu().numpy())
        res["cpu_baseline"] = {"value": round(bytes_["total"] / t_cpu / 1e9, 3), "unit": "GB/s", "cores": threads,
                               "kind": "port", "sample": "the full batch of this workload on the GPU leg's own inputs "
                               "(query, quantised caches and block table copied to the host), mean of %d passes of the "
                               "CPU checker over %.1f s (%.4f s per pass)" % (n_pass, n_pass * t_cpu, t_cpu),
                               "value_1_thread": round(bytes_["total"] / t_one / 1e9, 3), "cpu": cpu_model(),
                               "host_cpus": os.cpu_count()}
    print(json.dumps(res))


if __name__ == "__main__":
    main()
