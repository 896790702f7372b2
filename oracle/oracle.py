"""ctypes front end of the CPU checker in ``pa_oracle.cpp``.

TEST INFRASTRUCTURE ONLY: imported by ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline``
leg of ``bench.py``; the product package never imports it.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libpa_oracle.so")

DT_F16, DT_BF16, DT_U8, DT_U4 = 0, 1, 2, 3
MODE_SUM, MODE_NORM_SUM, MODE_ADAPTIVE_RKV = 0, 1, 2


def build(force=False):
    """Compiles the checker with the Makefile next to it."""
    if force and os.path.exists(_SO):
        os.remove(_SO)
    subprocess.check_call(["make", "-C", _HERE, "libpa_oracle.so"], stdout=subprocess.DEVNULL)


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        L = C.CDLL(_SO)
        L.orc_last_error.restype = C.c_char_p
        L.orc_half_to_float.restype = C.c_float
        L.orc_half_to_float.argtypes = [C.c_uint16]
        L.orc_float_to_half.restype = C.c_uint16
        L.orc_float_to_half.argtypes = [C.c_float]
        L.orc_bf16_to_float.restype = C.c_float
        L.orc_bf16_to_float.argtypes = [C.c_uint16]
        L.orc_float_to_bf16.restype = C.c_uint16
        L.orc_float_to_bf16.argtypes = [C.c_float]
        for name in ("orc_mgr_create", "orc_evict_create", "orc_evict_create_full", "orc_kvcrush_create"):
            getattr(L, name).restype = C.c_void_p
        L.orc_evict_create_full.argtypes = [C.c_uint64, C.c_uint64, C.c_uint64, C.c_int32, C.c_uint64, C.c_uint64,
                                            C.c_uint64, C.c_uint64, C.c_uint64, C.c_double, C.c_uint64, C.c_int32,
                                            C.c_uint64]
        L.orc_adaptive_rkv_diversity.argtypes = [C.c_void_p, C.c_int32, C.c_int64, C.c_int32, C.c_int32, C.c_int32,
                                                 C.POINTER(C.c_int32), C.c_int32, C.c_int32, C.c_int32,
                                                 C.POINTER(C.c_double), C.POINTER(C.c_double), C.c_double]
        L.orc_kvcrush_create.argtypes = [C.c_uint64, C.c_int32, C.c_uint64, C.c_uint64]
        L.orc_kvcrush_destroy.argtypes = [C.c_void_p]
        U64P, F64P = C.POINTER(C.c_uint64), C.POINTER(C.c_double)
        L.orc_rkv_diversity_block_set.restype = C.c_uint64
        L.orc_rkv_diversity_block_set.argtypes = [C.c_double, C.c_uint64, C.c_uint64, F64P, C.c_uint64, U64P, U64P]
        L.orc_rkv_filtered_block_diversity.argtypes = [C.c_uint64, F64P, C.c_uint64, C.c_uint64, U64P, C.c_uint64, F64P]
        L.orc_rkv_most_diverse_blocks.restype = C.c_uint64
        L.orc_rkv_most_diverse_blocks.argtypes = [C.c_uint64, U64P, C.c_uint64, F64P, U64P]
        L.orc_kvcrush_indicators.argtypes = [C.c_void_p, C.c_uint64, F64P, C.c_uint64, U64P]
        L.orc_kvcrush_anchor_point.argtypes = [C.c_void_p, C.c_uint64, U64P, U64P]
        L.orc_kvcrush_hamming.argtypes = [C.c_void_p, C.c_uint64, U64P, U64P, U64P]
        L.orc_kvcrush_representative.restype = C.c_uint64
        L.orc_kvcrush_representative.argtypes = [C.c_void_p, U64P, C.c_uint64, U64P, C.c_uint64, U64P]
        L.orc_kvcrush_blocks_to_retain.restype = C.c_uint64
        L.orc_kvcrush_blocks_to_retain.argtypes = [C.c_void_p, C.c_uint64, U64P, C.c_uint64, F64P, C.c_uint64, U64P]
        L.orc_mgr_create.argtypes = [C.c_uint64, C.c_uint64, C.c_uint64, C.c_int32, C.c_uint64, C.c_uint64, C.c_uint64]
        L.orc_evict_create.argtypes = [C.c_uint64, C.c_uint64, C.c_uint64, C.c_int32, C.c_uint64, C.c_uint64,
                                       C.c_uint64, C.c_uint64]
        for name in ("orc_mgr_len", "orc_mgr_counter_len", "orc_evict_len", "orc_evict_max_after",
                     "orc_evict_block_scores", "orc_evict_run", "orc_snapkv_num_scores"):
            getattr(L, name).restype = C.c_uint64
        L.orc_snapkv_num_scores.argtypes = [C.c_uint64] * 4
        L.orc_trishape_skipped_blocks.restype = C.c_int64
        L.orc_trishape_skipped_blocks.argtypes = [C.c_uint64] * 8 + [C.POINTER(C.c_uint64)]
        L.orc_rotation_luts.argtypes = [C.c_uint64, C.c_uint64, C.c_uint64, C.c_double, C.POINTER(C.c_float),
                                        C.POINTER(C.c_float)]
        L.orc_rotation_trig_lut.argtypes = [C.c_uint64, C.c_uint64, C.c_uint64, C.c_double, C.POINTER(C.c_float)]
        L.orc_rotation_data.restype = C.c_int64
        L.orc_rotation_data.argtypes = [C.POINTER(C.c_uint64), C.c_uint64, C.c_uint64, C.c_uint64, C.c_uint64,
                                        C.POINTER(C.c_uint64), C.POINTER(C.c_uint64), C.c_uint64]
        L.orc_rotate_cache.argtypes = [C.c_void_p, C.c_int32, C.c_int64, C.c_int32, C.c_int32, C.c_int32,
                                       C.POINTER(C.c_int32), C.c_int32, C.POINTER(C.c_int32), C.c_int32,
                                       C.POINTER(C.c_float), C.c_int32]
        _lib = L
    return _lib


def _ptr(a, t):
    return a.ctypes.data_as(C.POINTER(t)) if a is not None else None


def _err():
    return lib().orc_last_error().decode()


# ----------------------------------------------------------------------------- 16-bit float views
def f32_to_bf16_bits(x):
    """Round-to-nearest-even float32 -> bfloat16 bit patterns (uint16)."""
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32).astype(np.uint64)
    lsb = (u >> 16) & 1
    return ((u + 0x7FFF + lsb) >> 16).astype(np.uint16)


def bf16_bits_to_f32(b):
    return (np.ascontiguousarray(b, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


def to_bits(x_f32, dtype):
    """float32 array -> uint16 bit patterns of ``dtype`` (DT_F16 / DT_BF16)."""
    if dtype == DT_F16:
        return np.ascontiguousarray(x_f32, dtype=np.float32).astype(np.float16).view(np.uint16)
    return f32_to_bf16_bits(x_f32)


def from_bits(bits, dtype):
    if dtype == DT_F16:
        return np.ascontiguousarray(bits, dtype=np.uint16).view(np.float16).astype(np.float32)
    return bf16_bits_to_f32(bits)


# ----------------------------------------------------------------------------- KV rows
def quantize_row_u8(x):
    x = np.ascontiguousarray(x, dtype=np.float32)
    row = np.zeros(x.size + 8, dtype=np.uint8)
    lib().orc_quantize_row_u8(_ptr(x, C.c_float), C.c_int32(x.size), _ptr(row, C.c_uint8))
    return row


def quantize_row_u4(x):
    x = np.ascontiguousarray(x, dtype=np.float32)
    row = np.zeros(x.size // 2 + 8, dtype=np.uint8)
    lib().orc_quantize_row_u4(_ptr(x, C.c_float), C.c_int32(x.size), _ptr(row, C.c_uint8))
    return row


def row_bytes(D, cache_dtype):
    return D + 8 if cache_dtype == DT_U8 else D // 2 + 8 if cache_dtype == DT_U4 else 2 * D


def kv_append(key, value, src_dtype, key_cache, value_cache, cache_dtype, past_lens, subsequence_begins,
              block_indices, block_indices_begins, Hkv, D, bs):
    """key/value: uint16 [T, Hkv*D]; caches: uint8 [num_blocks, Hkv, bs, row_bytes], updated in place."""
    B = len(past_lens)
    nb = key_cache.shape[0]
    rc = lib().orc_kv_append(
        _ptr(key, C.c_uint16), _ptr(value, C.c_uint16), C.c_int32(src_dtype), _ptr(key_cache, C.c_uint8),
        _ptr(value_cache, C.c_uint8), C.c_int32(cache_dtype), C.c_int64(nb), _ptr(past_lens, C.c_int32),
        _ptr(subsequence_begins, C.c_int32), _ptr(block_indices, C.c_int32), _ptr(block_indices_begins, C.c_int32),
        C.c_int32(B), C.c_int32(Hkv), C.c_int32(D), C.c_int32(bs))
    if rc != 0:
        raise RuntimeError(_err())


def kv_append_kv(key, value, src_dtype, key_cache, value_cache, k_dtype, v_dtype, past_lens, subsequence_begins,
                 block_indices, block_indices_begins, Hkv, Dk, Dv, bs):
    """kv_append with a head size and an element type per tensor: key [T, Hkv*Dk], value [T, Hkv*Dv]."""
    rc = lib().orc_kv_append_kv(
        _ptr(key, C.c_uint16), _ptr(value, C.c_uint16), C.c_int32(src_dtype), _ptr(key_cache, C.c_uint8),
        _ptr(value_cache, C.c_uint8), C.c_int32(k_dtype), C.c_int32(v_dtype), C.c_int64(key_cache.shape[0]),
        _ptr(past_lens, C.c_int32), _ptr(subsequence_begins, C.c_int32), _ptr(block_indices, C.c_int32),
        _ptr(block_indices_begins, C.c_int32), C.c_int32(len(past_lens)), C.c_int32(Hkv), C.c_int32(Dk), C.c_int32(Dv),
        C.c_int32(bs))
    if rc != 0:
        raise RuntimeError(_err())


def paged_attention_kv(query, q_dtype, key_cache, value_cache, k_dtype, v_dtype, past_lens, subsequence_begins,
                       block_indices, block_indices_begins, Hq, Hkv, Dk, Dv, bs, scale, sliding_window=0,
                       score_aggregation_window=None, want_scores=True, num_threads=1):
    """paged_attention with a head size and an element type per tensor: query [T, Hq*Dk], out [T, Hq*Dv]."""
    B = len(past_lens)
    T = int(subsequence_begins[-1])
    out = np.zeros((T, Hq * Dv), dtype=np.float32)
    out16 = np.zeros((T, Hq * Dv), dtype=np.uint16)
    total = int(np.sum(past_lens.astype(np.int64)) + T)
    scores = np.zeros(total, dtype=np.float32) if want_scores else None
    saw = None if score_aggregation_window is None else np.ascontiguousarray(score_aggregation_window, dtype=np.int32)
    rc = lib().orc_paged_attention_kv(
        _ptr(query, C.c_uint16), C.c_int32(q_dtype), _ptr(key_cache, C.c_uint8), _ptr(value_cache, C.c_uint8),
        C.c_int32(k_dtype), C.c_int32(v_dtype), C.c_int64(key_cache.shape[0]), _ptr(past_lens, C.c_int32),
        _ptr(subsequence_begins, C.c_int32), _ptr(block_indices, C.c_int32), _ptr(block_indices_begins, C.c_int32),
        _ptr(saw, C.c_int32), C.c_int32(B), C.c_int32(Hq), C.c_int32(Hkv), C.c_int32(Dk), C.c_int32(Dv), C.c_int32(bs),
        C.c_float(scale), C.c_int32(sliding_window), _ptr(out, C.c_float), _ptr(out16, C.c_uint16),
        _ptr(scores, C.c_float), C.c_int32(num_threads))
    if rc != 0:
        raise RuntimeError(_err())
    return out, out16, scores


def paged_attention_alibi(query, q_dtype, key_cache, value_cache, k_dtype, v_dtype, past_lens, subsequence_begins,
                          block_indices, block_indices_begins, Hq, Hkv, Dk, Dv, bs, scale, alibi_slopes, sliding_window=0,
                          score_aggregation_window=None, want_scores=True, num_threads=1):
    """paged_attention_kv with the op's alibi_slopes input (f32 [Hq])."""
    B = len(past_lens)
    T = int(subsequence_begins[-1])
    out = np.zeros((T, Hq * Dv), dtype=np.float32)
    out16 = np.zeros((T, Hq * Dv), dtype=np.uint16)
    total = int(np.sum(past_lens.astype(np.int64)) + T)
    scores = np.zeros(total, dtype=np.float32) if want_scores else None
    saw = None if score_aggregation_window is None else np.ascontiguousarray(score_aggregation_window, dtype=np.int32)
    slopes = np.ascontiguousarray(alibi_slopes, dtype=np.float32)
    assert slopes.shape == (Hq,)
    rc = lib().orc_paged_attention_alibi(
        _ptr(query, C.c_uint16), C.c_int32(q_dtype), _ptr(key_cache, C.c_uint8), _ptr(value_cache, C.c_uint8),
        C.c_int32(k_dtype), C.c_int32(v_dtype), C.c_int64(key_cache.shape[0]), _ptr(past_lens, C.c_int32),
        _ptr(subsequence_begins, C.c_int32), _ptr(block_indices, C.c_int32), _ptr(block_indices_begins, C.c_int32),
        _ptr(saw, C.c_int32), C.c_int32(B), C.c_int32(Hq), C.c_int32(Hkv), C.c_int32(Dk), C.c_int32(Dv), C.c_int32(bs),
        C.c_float(scale), C.c_int32(sliding_window), _ptr(slopes, C.c_float), _ptr(out, C.c_float), _ptr(out16, C.c_uint16),
        _ptr(scores, C.c_float), C.c_int32(num_threads))
    if rc != 0:
        raise RuntimeError(_err())
    return out, out16, scores


def paged_attention(query, q_dtype, key_cache, value_cache, cache_dtype, past_lens, subsequence_begins,
                    block_indices, block_indices_begins, Hq, Hkv, D, bs, scale, sliding_window=0,
                    score_aggregation_window=None, want_scores=True, num_threads=1):
    """Returns (out_f32 [T, Hq*D], out16 bits [T, Hq*D], scores f32 or None)."""
    B = len(past_lens)
    T = int(subsequence_begins[-1])
    out = np.zeros((T, Hq * D), dtype=np.float32)
    out16 = np.zeros((T, Hq * D), dtype=np.uint16)
    total = int(np.sum(past_lens.astype(np.int64)) + T)
    scores = np.zeros(total, dtype=np.float32) if want_scores else None
    saw = None if score_aggregation_window is None else np.ascontiguousarray(score_aggregation_window, dtype=np.int32)
    rc = lib().orc_paged_attention(
        _ptr(query, C.c_uint16), C.c_int32(q_dtype), _ptr(key_cache, C.c_uint8), _ptr(value_cache, C.c_uint8),
        C.c_int32(cache_dtype), C.c_int64(key_cache.shape[0]), _ptr(past_lens, C.c_int32),
        _ptr(subsequence_begins, C.c_int32), _ptr(block_indices, C.c_int32), _ptr(block_indices_begins, C.c_int32),
        _ptr(saw, C.c_int32), C.c_int32(B), C.c_int32(Hq), C.c_int32(Hkv), C.c_int32(D), C.c_int32(bs),
        C.c_float(scale), C.c_int32(sliding_window), _ptr(out, C.c_float), _ptr(out16, C.c_uint16),
        _ptr(scores, C.c_float), C.c_int32(num_threads))
    if rc != 0:
        raise RuntimeError(_err())
    return out, out16, scores


def pack_step(processed, evicted, skipped_blocks, scheduled, num_blocks, bs):
    B = len(processed)
    a = [np.ascontiguousarray(v, dtype=np.int64) for v in (processed, evicted, skipped_blocks, scheduled, num_blocks)]
    past = np.zeros(B, np.int32)
    sb = np.zeros(B + 1, np.int32)
    bib = np.zeros(B + 1, np.int32)
    mx = C.c_int32(0)
    lib().orc_pack_step(C.c_int32(B), *[_ptr(v, C.c_int64) for v in a], C.c_int32(bs), _ptr(past, C.c_int32),
                        _ptr(sb, C.c_int32), _ptr(bib, C.c_int32), C.byref(mx))
    return past, sb, bib, mx.value


def normalize_num_kv_blocks(num_kv_blocks, cache_size_gib, block_size, block_bytes_all_layers, total_memory):
    out = C.c_uint64(0)
    rc = lib().orc_normalize_num_kv_blocks(C.c_uint64(num_kv_blocks), C.c_uint64(cache_size_gib),
                                           C.c_uint64(block_size), C.c_uint64(block_bytes_all_layers),
                                           C.c_uint64(total_memory), C.byref(out))
    if rc != 0:
        raise RuntimeError(_err())
    return out.value


def snapkv_num_scores(window, prompt_len, num_scheduled, num_processed):
    return int(lib().orc_snapkv_num_scores(window, prompt_len, num_scheduled, num_processed))


# ----------------------------------------------------------------------------- eviction
def _layer_args(layer_scores):
    arrs = [np.ascontiguousarray(s, dtype=np.float32) for s in layer_scores]
    ptrs = (C.POINTER(C.c_float) * len(arrs))(*[_ptr(a, C.c_float) for a in arrs])
    lens = np.array([a.size for a in arrs], dtype=np.uint64)
    return arrs, ptrs, lens


class ScoreManager:
    """Handle on the restated EvictionScoreManager."""

    def __init__(self, block_size, num_layers, max_pool_window_size, mode, ignore_first_n_blocks=0,
                 snapkv_window_size=0, adaptive_rkv_window_size=8):
        self.layers = num_layers
        self.h = C.c_void_p(lib().orc_mgr_create(block_size, num_layers, max_pool_window_size, mode,
                                                 ignore_first_n_blocks, snapkv_window_size, adaptive_rkv_window_size))

    def __del__(self):
        if getattr(self, "h", None) and lib is not None:  # module globals are gone at interpreter exit
            lib().orc_mgr_destroy(self.h)
            self.h = None

    def register_new_token_scores(self, layer_scores, skipped=(), num_snapkv_scores=0):
        arrs, ptrs, lens = _layer_args(layer_scores)
        sk = np.array(sorted(skipped), dtype=np.uint64)
        rc = lib().orc_mgr_register(self.h, ptrs, _ptr(lens, C.c_uint64), _ptr(sk, C.c_uint64), C.c_uint64(sk.size),
                                    C.c_uint64(num_snapkv_scores))
        if rc != 0:
            raise RuntimeError(_err())

    def remove_scores(self, evicted, layer):
        ev = np.array(list(evicted), dtype=np.uint64)
        lib().orc_mgr_remove(self.h, _ptr(ev, C.c_uint64), C.c_uint64(ev.size), C.c_uint64(layer))

    def get_scores(self):
        out = []
        for l in range(self.layers):
            s = np.zeros(lib().orc_mgr_len(self.h, C.c_uint64(l)), dtype=np.float64)
            lib().orc_mgr_get(self.h, C.c_uint64(l), _ptr(s, C.c_double), None)
            out.append(s)
        return out

    def get_counters(self):
        out = []
        for l in range(self.layers):
            c = np.zeros(lib().orc_mgr_counter_len(self.h, C.c_uint64(l)), dtype=np.uint64)
            lib().orc_mgr_get(self.h, C.c_uint64(l), None, _ptr(c, C.c_uint64))
            out.append(c)
        return out


def add_with_skips(block_size, dst, src, skipped):
    d = np.array(dst, dtype=np.float64)
    s = np.array(src, dtype=np.float64)
    sk = np.array(sorted(skipped), dtype=np.uint64)
    rc = lib().orc_add_with_skips(C.c_uint64(block_size), _ptr(d, C.c_double), C.c_uint64(d.size),
                                  _ptr(s, C.c_double), C.c_uint64(s.size), _ptr(sk, C.c_uint64), C.c_uint64(sk.size))
    if rc != 0:
        raise RuntimeError(_err())
    return d


ANCHOR_RANDOM, ANCHOR_ZEROS, ANCHOR_ONES, ANCHOR_MEAN, ANCHOR_ALTERNATING = range(5)


class CacheEvictionAlgorithm:
    """Handle on the restated CacheEvictionAlgorithm."""

    def __init__(self, start_size, recent_size, max_cache_size, mode, snapkv_window_size, block_size, num_layers,
                 max_pool_window_size, adaptive_rkv_window_size=8, attention_mass=0.9, kvcrush_budget=0,
                 kvcrush_anchor_mode=ANCHOR_RANDOM, kvcrush_seed=0):
        self.layers = num_layers
        h = lib().orc_evict_create_full(start_size, recent_size, max_cache_size, mode, snapkv_window_size, block_size,
                                        num_layers, max_pool_window_size, adaptive_rkv_window_size,
                                        float(attention_mass), kvcrush_budget, kvcrush_anchor_mode, kvcrush_seed)
        if not h:
            raise ValueError(_err())
        self.h = C.c_void_p(h)

    def __del__(self):
        if getattr(self, "h", None) and lib is not None:
            lib().orc_evict_destroy(self.h)
            self.h = None

    def get_max_cache_size_after_eviction(self):
        return int(lib().orc_evict_max_after(self.h))

    def register_new_token_scores(self, layer_scores, skipped=(), num_snapkv_scores=0):
        arrs, ptrs, lens = _layer_args(layer_scores)
        sk = np.array(sorted(skipped), dtype=np.uint64)
        rc = lib().orc_evict_register(self.h, ptrs, _ptr(lens, C.c_uint64), _ptr(sk, C.c_uint64),
                                      C.c_uint64(sk.size), C.c_uint64(num_snapkv_scores))
        if rc != 0:
            raise RuntimeError(_err())

    def get_evictable_block_range(self, layer=0):
        b, e = C.c_uint64(0), C.c_uint64(0)
        lib().orc_evict_range(self.h, C.c_uint64(layer), C.byref(b), C.byref(e))
        return b.value, e.value

    def block_scores(self, layer):
        cap = 1 << 16
        out = np.zeros(cap, dtype=np.float64)
        n = int(lib().orc_evict_block_scores(self.h, C.c_uint64(layer), _ptr(out, C.c_double), C.c_uint64(cap)))
        return out[:n].copy()

    def register_block_diversity(self, layer_diversity):
        arrs, ptrs, lens = _layer_args(layer_diversity)
        if lib().orc_evict_register_diversity(self.h, ptrs, _ptr(lens, C.c_uint64)) != 0:
            raise RuntimeError(_err())

    def evict_logical_blocks(self):
        cap = 1 << 20
        blocks = np.zeros(cap, dtype=np.uint64)
        counts = np.zeros(self.layers, dtype=np.uint64)
        n = lib().orc_evict_run(self.h, _ptr(blocks, C.c_uint64), C.c_uint64(cap), _ptr(counts, C.c_uint64))
        if n == 2**64 - 1:
            raise RuntimeError(_err())
        out, o = [], 0
        for l in range(self.layers):
            out.append([int(v) for v in blocks[o:o + int(counts[l])]])
            o += int(counts[l])
        return out

    def get_scores(self):
        out = []
        for l in range(self.layers):
            s = np.zeros(lib().orc_evict_len(self.h, C.c_uint64(l)), dtype=np.float64)
            lib().orc_evict_get(self.h, C.c_uint64(l), _ptr(s, C.c_double), None)
            out.append(s)
        return out

    def get_counters(self, norm_sum=True):
        out = []
        for l in range(self.layers):
            n = lib().orc_evict_len(self.h, C.c_uint64(l)) if norm_sum else 0
            c = np.zeros(n, dtype=np.uint64)
            lib().orc_evict_get(self.h, C.c_uint64(l), None, _ptr(c, C.c_uint64))
            out.append(c)
        return out


def adaptive_rkv_diversity(key_cache, cache_dtype, Hkv, bs, D, table, start_size, evictable_size, margin=0.0):
    """Block diversity of one sequence's evictable area: ([ev / bs, ev] values, same-shape slack for entries within
    ``margin`` of their row's mean).  PARITY UNPINNED, see pa_oracle.cpp."""
    kc = np.ascontiguousarray(key_cache)
    t = np.ascontiguousarray(table, np.int32)
    nb = evictable_size // bs
    out = np.zeros((nb, evictable_size), np.float64)
    slack = np.zeros((nb, evictable_size), np.float64)
    rc = lib().orc_adaptive_rkv_diversity(kc.ctypes.data_as(C.c_void_p), cache_dtype, kc.shape[0], Hkv, bs, D,
                                          _ptr(t, C.c_int32), t.size, start_size, evictable_size,
                                          _ptr(out, C.c_double), _ptr(slack, C.c_double), float(margin))
    if rc != 0:
        raise ValueError(_err())
    return out, slack


class AdaptiveRKVBlockCalculator:
    """Restatement of ``AdaptiveRKVBlockCalculator`` (cache_eviction.hpp, cache_eviction.cpp:659-737)."""

    def __init__(self, attention_mass, block_size):
        self.mass, self.block = float(attention_mass), int(block_size)

    def get_diversity_block_set(self, max_num_blocks_kept, block_scores):
        sc = np.ascontiguousarray(block_scores, dtype=np.float64)
        out = np.zeros(max(1, sc.size), np.uint64)
        kept = C.c_uint64(0)
        n = lib().orc_rkv_diversity_block_set(self.mass, self.block, max_num_blocks_kept, _ptr(sc, C.c_double), sc.size,
                                              _ptr(out, C.c_uint64), C.byref(kept))
        return set(int(v) for v in out[:n]), int(kept.value)

    def get_filtered_block_diversity(self, unfiltered, eviction_size, diversity_blocks):
        u = np.ascontiguousarray(unfiltered, dtype=np.float64)
        st = np.asarray(sorted(diversity_blocks), np.uint64)
        out = np.zeros(max(1, eviction_size // self.block), np.float64)
        if lib().orc_rkv_filtered_block_diversity(self.block, _ptr(u, C.c_double), u.size, eviction_size,
                                                  _ptr(st, C.c_uint64), st.size, _ptr(out, C.c_double)) != 0:
            raise ValueError(_err())
        return out[:eviction_size // self.block]

    def get_most_diverse_blocks(self, num_blocks_left_to_fill, diversity_blocks, filtered):
        st = np.asarray(sorted(diversity_blocks), np.uint64)
        f = np.ascontiguousarray(filtered, dtype=np.float64)
        out = np.zeros(max(1, st.size), np.uint64)
        n = lib().orc_rkv_most_diverse_blocks(num_blocks_left_to_fill, _ptr(st, C.c_uint64), st.size,
                                              _ptr(f, C.c_double), _ptr(out, C.c_uint64))
        return set(int(v) for v in out[:n])


class KVCrushAlgorithm:
    """Restatement of ``KVCrushAlgorithm`` (kvcrush.hpp, kvcrush.cpp:9-174)."""

    def __init__(self, budget, anchor_point_mode, rng_seed, block_size):
        self.block = int(block_size)
        self.h = C.c_void_p(lib().orc_kvcrush_create(budget, anchor_point_mode, rng_seed, block_size))

    def __del__(self):
        if getattr(self, "h", None) and lib is not None:
            lib().orc_kvcrush_destroy(self.h)
            self.h = None

    def create_indicators(self, num_tokens, layer_scores):
        sc = np.ascontiguousarray(layer_scores, dtype=np.float64)
        out = np.zeros(max(1, num_tokens), np.uint64)
        lib().orc_kvcrush_indicators(self.h, num_tokens, _ptr(sc, C.c_double), sc.size, _ptr(out, C.c_uint64))
        return [int(v) for v in out[:num_tokens]]

    def create_anchor_point(self, num_tokens, indicators):
        ind = np.asarray(indicators, np.uint64)
        out = np.zeros(self.block, np.uint64)
        if lib().orc_kvcrush_anchor_point(self.h, num_tokens, _ptr(ind, C.c_uint64), _ptr(out, C.c_uint64)) != 0:
            raise ValueError(_err())
        return [int(v) for v in out]

    def calculate_hamming_distance(self, num_tokens, indicators, anchor_point):
        ind = np.asarray(indicators, np.uint64)
        an = np.asarray(anchor_point, np.uint64)
        out = np.zeros(max(1, num_tokens // self.block), np.uint64)
        lib().orc_kvcrush_hamming(self.h, num_tokens, _ptr(ind, C.c_uint64), _ptr(an, C.c_uint64), _ptr(out, C.c_uint64))
        return [int(v) for v in out[:num_tokens // self.block]]

    def get_representative_blocks(self, distances, eligible):
        d = np.asarray(distances, np.uint64)
        el = np.asarray(eligible, np.uint64)
        out = np.zeros(max(1, d.size), np.uint64)
        n = lib().orc_kvcrush_representative(self.h, _ptr(d, C.c_uint64), d.size, _ptr(el, C.c_uint64), el.size,
                                             _ptr(out, C.c_uint64))
        return [int(v) for v in out[:n]]

    def get_indices_of_blocks_to_retain(self, num_tokens, evicted, layer_scores):
        ev = np.asarray(evicted, np.uint64)
        sc = np.ascontiguousarray(layer_scores, dtype=np.float64)
        out = np.zeros(max(1, ev.size), np.uint64)
        n = lib().orc_kvcrush_blocks_to_retain(self.h, num_tokens, _ptr(ev, C.c_uint64), ev.size, _ptr(sc, C.c_double),
                                               sc.size, _ptr(out, C.c_uint64))
        return [int(v) for v in out[:n]]


# ----------------------------------------------------------------------------- cache rotation
class CacheRotationCalculator:
    """Restatement of ``CacheRotationCalculator`` (cache_eviction.hpp:262-335, cache_eviction.cpp:543-636)."""

    def __init__(self, block_size, max_context_length_in_blocks, kv_head_size, rope_theta=10000.0):
        self.block_size, self.max_blocks, self.head_size = block_size, max_context_length_in_blocks, kv_head_size
        nf = kv_head_size // 2
        self.sin_lut = np.zeros((max_context_length_in_blocks, nf), np.float32)
        self.cos_lut = np.zeros((max_context_length_in_blocks, nf), np.float32)
        if lib().orc_rotation_luts(block_size, max_context_length_in_blocks, kv_head_size, float(rope_theta),
                                   _ptr(self.sin_lut, C.c_float), _ptr(self.cos_lut, C.c_float)):
            raise ValueError(_err())

    def get_rotation_data(self, evicted_block_logical_indices, num_logical_blocks_before_eviction, deltas_only=True):
        """List of dicts: logical_block_idx (after eviction), rotation_delta (tokens) [, sines, cosines per token]."""
        ev = np.asarray(sorted(set(int(v) for v in evicted_block_logical_indices)), np.uint64)
        cap = max(1, int(num_logical_blocks_before_eviction))
        idx = np.zeros(cap, np.uint64)
        delta = np.zeros(cap, np.uint64)
        n = lib().orc_rotation_data(_ptr(ev, C.c_uint64) if len(ev) else None, len(ev),
                                    int(num_logical_blocks_before_eviction), self.block_size, self.max_blocks,
                                    _ptr(idx, C.c_uint64), _ptr(delta, C.c_uint64), cap)
        if n < 0:
            raise ValueError(_err())
        out = []
        for i in range(n):
            d = dict(logical_block_idx=int(idx[i]), rotation_delta=int(delta[i]))
            if not deltas_only:
                row = int(delta[i]) // self.block_size
                d["sines"] = [self.sin_lut[row].copy() for _ in range(self.block_size)]
                d["cosines"] = [self.cos_lut[row].copy() for _ in range(self.block_size)]
            out.append(d)
        return out


def rotation_trig_lut(block_size, max_blocks, head_size, rope_theta=10000.0):
    lut = np.zeros((max_blocks, head_size), np.float32)
    if lib().orc_rotation_trig_lut(block_size, max_blocks, head_size, float(rope_theta), _ptr(lut, C.c_float)):
        raise ValueError(_err())
    return lut


def rotate_cache(key_cache, cache_dtype, rotated_block_indices, rotation_deltas, trig_lut):
    """In-place re-rotation of the K rows of the listed physical blocks; ``rotation_deltas`` is [n, 1] or [n, bs]."""
    num_blocks, Hkv, bs, rb = key_cache.shape
    D = rb - 8 if cache_dtype == DT_U8 else rb // 2
    idx = np.ascontiguousarray(rotated_block_indices, np.int32)
    dl = np.ascontiguousarray(rotation_deltas, np.int32).reshape(len(idx), -1)
    lut = np.ascontiguousarray(trig_lut, np.float32)
    rc = lib().orc_rotate_cache(key_cache.ctypes.data_as(C.c_void_p), cache_dtype, num_blocks, Hkv, bs, D,
                                _ptr(idx, C.c_int32), len(idx), _ptr(dl, C.c_int32), dl.shape[1],
                                _ptr(lut, C.c_float), lut.shape[0])
    if rc:
        raise ValueError(_err())


# ----------------------------------------------------------------------------- sparse prefill
def trishape_skipped_blocks(block_size, num_last_dense_tokens_in_prefill, num_retained_start_tokens_in_cache,
                            num_retained_recent_tokens_in_cache, prompt_len, num_processed_tokens,
                            num_scheduled_tokens, num_cached_tokens=None):
    """Set of logical blocks TriShapeSparseAttentionTokenSkipper skips for the next inference of a sequence group."""
    first = C.c_uint64(0)
    cached = num_processed_tokens if num_cached_tokens is None else num_cached_tokens
    n = lib().orc_trishape_skipped_blocks(block_size, num_last_dense_tokens_in_prefill,
                                          num_retained_start_tokens_in_cache, num_retained_recent_tokens_in_cache,
                                          prompt_len, num_processed_tokens, num_scheduled_tokens, cached, C.byref(first))
    if n < 0:
        raise ValueError(_err())
    return set(range(first.value, first.value + n))


# ----------------------------------------------------------------------------- XAttention (sparse prefill)
def xattention_shape(past, q_len, xb):
    """(first query block, query blocks the chunk touches, key blocks) of a sequence."""
    qb0 = past // xb
    nkb = (past + q_len - 1) // xb + 1
    return qb0, nkb - qb0, nkb


def xattention_block_sums(query, q_dtype, key_cache, cache_dtype, table, tok0, past, q_len, Hq, Hkv, D, bs, scale, xb,
                          stride):
    """Block sums of the antidiagonal importance estimate of one sequence: float64 [Hq, nqb, nkb]."""
    _, nqb, nkb = xattention_shape(past, q_len, xb)
    sums = np.zeros((Hq, nqb, nkb), dtype=np.float64)
    table = np.ascontiguousarray(table, dtype=np.int32)
    rc = lib().orc_xattention_block_sums(
        _ptr(query, C.c_uint16), C.c_int32(q_dtype), _ptr(key_cache, C.c_uint8), C.c_int32(cache_dtype),
        C.c_int64(key_cache.shape[0]), _ptr(table, C.c_int32), C.c_int32(len(table)), C.c_int32(tok0), C.c_int32(past),
        C.c_int32(q_len), C.c_int32(Hq), C.c_int32(Hkv), C.c_int32(D), C.c_int32(bs), C.c_float(scale), C.c_int32(xb),
        C.c_int32(stride), _ptr(sums, C.c_double))
    if rc != 0:
        raise RuntimeError(_err())
    return sums


def xattention_select(sums, qb0, threshold):
    """(retained uint8 [Hq, nqb, nkb], slack float64 [Hq, nqb]) for block sums [Hq, nqb, nkb]."""
    sums = np.ascontiguousarray(sums, dtype=np.float64)
    Hq, nqb, nkb = sums.shape
    retained = np.zeros((Hq, nqb, nkb), dtype=np.uint8)
    slack = np.zeros((Hq, nqb), dtype=np.float64)
    rc = lib().orc_xattention_select(_ptr(sums, C.c_double), C.c_int32(Hq), C.c_int32(nqb), C.c_int32(nkb),
                                     C.c_int32(qb0), C.c_double(float(np.float32(threshold))), _ptr(retained, C.c_uint8),
                                     _ptr(slack, C.c_double))
    if rc != 0:
        raise RuntimeError(_err())
    return retained, slack


def paged_attention_sparse(query, q_dtype, key_cache, value_cache, cache_dtype, past_lens, subsequence_begins,
                           block_indices, block_indices_begins, Hq, Hkv, D, bs, scale, retained, xb, sliding_window=0,
                           score_aggregation_window=None, want_scores=True, num_threads=1):
    """paged_attention with per-sequence block masks: retained[b] is None or uint8 [Hq, nqb_b, nkb_b]."""
    B = len(past_lens)
    T = int(subsequence_begins[-1])
    out = np.zeros((T, Hq * D), dtype=np.float32)
    out16 = np.zeros((T, Hq * D), dtype=np.uint16)
    total = int(np.sum(past_lens.astype(np.int64)) + T)
    scores = np.zeros(total, dtype=np.float32) if want_scores else None
    saw = None if score_aggregation_window is None else np.ascontiguousarray(score_aggregation_window, dtype=np.int32)
    keep = [None if r is None else np.ascontiguousarray(r, dtype=np.uint8) for r in retained]
    ptrs = (C.c_void_p * B)(*[None if r is None else r.ctypes.data for r in keep])
    rc = lib().orc_paged_attention_sparse(
        _ptr(query, C.c_uint16), C.c_int32(q_dtype), _ptr(key_cache, C.c_uint8), _ptr(value_cache, C.c_uint8),
        C.c_int32(cache_dtype), C.c_int64(key_cache.shape[0]), _ptr(past_lens, C.c_int32),
        _ptr(subsequence_begins, C.c_int32), _ptr(block_indices, C.c_int32), _ptr(block_indices_begins, C.c_int32),
        _ptr(saw, C.c_int32), C.c_int32(B), C.c_int32(Hq), C.c_int32(Hkv), C.c_int32(D), C.c_int32(bs),
        C.c_float(scale), C.c_int32(sliding_window), _ptr(out, C.c_float), _ptr(out16, C.c_uint16),
        _ptr(scores, C.c_float), C.c_int32(num_threads), ptrs, C.c_int32(xb))
    if rc != 0:
        raise RuntimeError(_err())
    return out, out16, scores


def xattention_threshold(configured, num_last_dense_tokens_in_prefill, prompt_len, num_processed_tokens,
                         num_scheduled_tokens, can_generate_tokens):
    f = lib().orc_xattention_threshold
    f.restype = C.c_float
    return float(f(C.c_float(configured), C.c_uint64(num_last_dense_tokens_in_prefill), C.c_uint64(prompt_len),
                   C.c_uint64(num_processed_tokens), C.c_uint64(num_scheduled_tokens), C.c_int32(int(can_generate_tokens))))
