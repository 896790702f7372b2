"""The PagedAttention op behind its reference input contract.

Inputs keep the names ModelRunner::forward binds on the infer request
(src/cpp/src/continuous_batching/model_runner.hpp:505-522, 907-948): ``past_lens``, ``subsequence_begins``,
``block_indices``, ``block_indices_begins``, ``max_context_len``, ``score_aggregation_window``; ``scale`` and
``sliding_window`` are the op's constants.  Tensors are torch CUDA tensors used only as device memory.
"""
import ctypes as C

import numpy as np

from . import _lib as L

_DTYPES = {"f16": L.PA_F16, "bf16": L.PA_BF16, "u8": L.PA_U8, "u4": L.PA_U4}


def dtype_code(name):
    return _DTYPES[name] if isinstance(name, str) else int(name)


def row_bytes(head_size, kv_cache_dtype):
    """Bytes of one cached row: 16-bit values, or `f32 scale | f32 zero-point` and the codes (u8: one byte each, u4: two per byte)."""
    dt = dtype_code(kv_cache_dtype)
    return head_size + 8 if dt == L.PA_U8 else head_size // 2 + 8 if dt == L.PA_U4 else 2 * head_size


def _i32(a):
    return np.ascontiguousarray(a, dtype=np.int32)


def _p32(a):
    return a.ctypes.data_as(C.POINTER(C.c_int32))


class PagedAttention:
    def __init__(self, num_heads, num_kv_heads, head_size, block_size=32, query_dtype="f16", kv_cache_dtype="u8",
                 num_layers=1, device=0, stream=None, v_head_size=None, value_cache_dtype=None):
        """``v_head_size`` / ``value_cache_dtype``: head size and precision of ``value_cache.<L>`` where they differ
        from the key side's (``head_size`` / ``kv_cache_dtype``)."""
        cfg = L.pa_config()
        cfg.device, cfg.num_heads, cfg.num_kv_heads, cfg.head_size = device, num_heads, num_kv_heads, head_size
        cfg.block_size, cfg.query_dtype, cfg.kv_cache_dtype = block_size, dtype_code(query_dtype), dtype_code(kv_cache_dtype)
        cfg.num_layers = num_layers
        cfg.v_head_size = 0 if v_head_size is None else int(v_head_size)
        cfg.value_cache_dtype_p1 = 0 if value_cache_dtype is None else 1 + dtype_code(value_cache_dtype)
        cfg.stream = C.c_void_p(int(getattr(stream, "cuda_stream", stream))) if stream is not None else None
        self.cfg = cfg
        h = C.c_void_p()
        L.check(L.lib().pa_create(C.byref(cfg), C.byref(h)), None)
        self._h = h
        self._keep = None

    def __del__(self):
        if getattr(self, "_h", None) and L is not None:  # module globals are gone at interpreter exit
            L.lib().pa_destroy(self._h)
            self._h = None

    def _ck(self, status):
        L.check(status, L.lib().pa_last_error, self._h)

    def step_begin(self, past_lens, subsequence_begins, block_indices_begins, max_context_len=0,
                   score_aggregation_window=None, sliding_window=0, scale=0.0):
        m = L.pa_step_meta()
        past, sb, bib = _i32(past_lens), _i32(subsequence_begins), _i32(block_indices_begins)
        saw = _i32(score_aggregation_window) if score_aggregation_window is not None else None
        m.num_sequences = len(past)
        m.past_lens, m.subsequence_begins, m.block_indices_begins = _p32(past), _p32(sb), _p32(bib)
        m.score_aggregation_window = _p32(saw) if saw is not None else None
        m.max_context_len, m.sliding_window, m.scale = int(max_context_len), int(sliding_window), float(scale)
        self._ck(L.lib().pa_step_begin(self._h, C.byref(m)))
        self.total_scores = int(np.sum(past.astype(np.int64)) + sb[-1])
        self.num_tokens = int(sb[-1])

    def set_block_indices(self, block_indices, num_blocks, layer=-1):
        ids = _i32(block_indices)
        self._ck(L.lib().pa_set_block_indices(self._h, layer, _p32(ids), len(ids), int(num_blocks)))

    def set_alibi_slopes(self, slopes):
        """The op's `alibi_slopes` input: one f32 slope per query head (None or empty: no ALiBi term).  Call before
        ``step_begin``; a context with slopes runs on the shape-generic kernels."""
        a = np.ascontiguousarray(slopes if slopes is not None else [], dtype=np.float32)
        self._ck(L.lib().pa_set_alibi_slopes(self._h, a.ctypes.data_as(C.POINTER(C.c_float)), len(a)))

    def set_block_indices_per_layer(self, tables, num_blocks, first_layer=0):
        """`block_indices.<L>` of layers first_layer .. first_layer + len(tables) - 1 in one call."""
        arrs = [_i32(t) for t in tables]
        n = len(arrs[0]) if arrs else 0
        if any(len(a) != n for a in arrs):
            raise ValueError("every layer's block_indices must have the same length")
        ptrs = (C.POINTER(C.c_int32) * len(arrs))(*[_p32(a) for a in arrs])
        self._ck(L.lib().pa_set_block_indices_layers(self._h, int(first_layer), len(arrs), ptrs, n, int(num_blocks)))

    def _io(self, query, key, value, key_cache, value_cache, out, scores):
        io = L.pa_layer_io()
        ptr = lambda t: C.c_void_p(t.data_ptr()) if t is not None else None
        io.query, io.key, io.value = ptr(query), ptr(key), ptr(value)
        io.key_cache, io.value_cache, io.num_blocks = ptr(key_cache), ptr(value_cache), key_cache.shape[0]
        io.out, io.scores = ptr(out), ptr(scores)
        return io

    def kv_append(self, key, value, key_cache, value_cache, layer=0):
        io = self._io(None, key, value, key_cache, value_cache, None, None)
        self._ck(L.lib().pa_kv_append(self._h, layer, C.byref(io)))

    def attention(self, query, key_cache, value_cache, out, scores=None, layer=0):
        io = self._io(query, None, None, key_cache, value_cache, out, scores)
        self._ck(L.lib().pa_attention(self._h, layer, C.byref(io)))

    def attention_static(self, query, key_cache, value_cache, out, scores=None, layer=0):
        """``attention`` without any allocation inside the call: workspaces come from the library's fixed device
        scratch (single-token steps only; a step that needs more than the scratch holds raises OUT_OF_BOUNDS)."""
        io = self._io(query, None, None, key_cache, value_cache, out, scores)
        self._ck(L.lib().pa_attention_static(self._h, layer, C.byref(io)))

    def forward(self, query, key, value, key_cache, value_cache, out, scores=None, layer=0):
        io = self._io(query, key, value, key_cache, value_cache, out, scores)
        self._ck(L.lib().pa_forward(self._h, layer, C.byref(io)))

    def synchronize(self):
        self._ck(L.lib().pa_synchronize(self._h))

    def set_profiling(self, enable=True):
        self._ck(L.lib().pa_set_profiling(self._h, 1 if enable else 0))

    def last_kernel_ms(self):
        ms = C.c_float(0.0)
        self._ck(L.lib().pa_last_kernel_ms(self._h, C.byref(ms)))
        return ms.value

    def set_rotation_trig_lut(self, lut):
        """Uploads the [rows, head_size] table of cosines | negated sines (the `model_rotation_trig_lut` input)."""
        lut = np.ascontiguousarray(lut, np.float32)
        self._ck(L.lib().pa_set_rotation_trig_lut(self._h, lut.ctypes.data_as(C.POINTER(C.c_float)), lut.shape[0]))

    def rotate_cache(self, key_cache, rotated_block_indices, rotation_deltas):
        """Re-rotates the K rows of the listed physical blocks in place (`rotated_block_indices.<L>`,
        `rotation_deltas.<L>` of shape [n, 1] or [n, block_size], values = table rows)."""
        idx = np.ascontiguousarray(rotated_block_indices, np.int32)
        deltas = np.ascontiguousarray(rotation_deltas, np.int32).reshape(len(idx), -1) if len(idx) else np.zeros((0, 1), np.int32)
        self._ck(L.lib().pa_rotate_cache(self._h, key_cache.data_ptr(), key_cache.shape[0], _p32(idx), len(idx),
                                         _p32(deltas), deltas.shape[1]))

    def adaptive_rkv_diversity(self, key_cache, start_size, evictable_sizes, diversity, layer=0):
        """Fills ``diversity`` (a device f32 tensor) with the `adaptive_rkv_diversity.<L>` output: for each sequence
        with a non-zero evictable size, its [evictable / block_size, evictable] matrix, concatenated in step order.
        Returns the B + 1 offsets of the sequences' spans."""
        ev = _i32(evictable_sizes)
        offsets = np.zeros(len(ev) + 1, np.int64)
        self._ck(L.lib().pa_adaptive_rkv_diversity(self._h, layer, C.c_void_p(key_cache.data_ptr()), key_cache.shape[0],
                                                   int(start_size), _p32(ev), C.c_void_p(diversity.data_ptr()),
                                                   diversity.numel(), offsets.ctypes.data_as(C.POINTER(C.c_int64))))
        return offsets

    def set_xattention(self, thresholds, xattention_block_size=64, xattention_stride=8):
        """``xattention_threshold.<L>`` (one value per sequence of the step), ``xattention_block_size``,
        ``xattention_stride`` (model_runner.hpp:1623-1656).  Call between ``step_begin`` and the layer calls."""
        if thresholds is None:
            self._ck(L.lib().pa_set_xattention(self._h, None, int(xattention_block_size), int(xattention_stride)))
            return
        thr = np.ascontiguousarray(thresholds, dtype=np.float32)
        self._ck(L.lib().pa_set_xattention(self._h, thr.ctypes.data_as(C.POINTER(C.c_float)), int(xattention_block_size),
                                           int(xattention_stride)))

    def xattention_shape(self, sequence):
        """(first query block, query blocks, key blocks) of a sequence of the step; zeros when it runs dense."""
        a, b, c = C.c_int32(0), C.c_int32(0), C.c_int32(0)
        self._ck(L.lib().pa_xattention_shape(self._h, int(sequence), C.byref(a), C.byref(b), C.byref(c)))
        return a.value, b.value, c.value

    def xattention_block_sums(self, sequence):
        """Block importances of the last layer call: float32 [num_heads, query blocks, key blocks]."""
        _, nqb, nkb = self.xattention_shape(sequence)
        out = np.zeros((self.cfg.num_heads, nqb, nkb), dtype=np.float32)
        self._ck(L.lib().pa_xattention_block_sums(self._h, int(sequence), out.ctypes.data_as(C.POINTER(C.c_float))))
        return out

    def xattention_retained(self, sequence):
        """Kept (query block, key block) pairs of the last layer call: uint8 [num_heads, query blocks, key blocks]."""
        _, nqb, nkb = self.xattention_shape(sequence)
        out = np.zeros((self.cfg.num_heads, nqb, nkb), dtype=np.uint8)
        self._ck(L.lib().pa_xattention_retained(self._h, int(sequence), out.ctypes.data_as(C.POINTER(C.c_uint8))))
        return out

    @property
    def num_splits(self):
        return int(L.lib().pa_get_num_splits(self._h))


def pack_step(processed, evicted, skipped_blocks, scheduled, num_blocks, block_size):
    """Integer part of ModelRunner::forward: returns past_lens, subsequence_begins, block_indices_begins, max_context_len."""
    B = len(processed)
    arrs = [np.ascontiguousarray(a, dtype=np.int64) for a in (processed, evicted, skipped_blocks, scheduled, num_blocks)]
    past, sb, bib = np.zeros(B, np.int32), np.zeros(B + 1, np.int32), np.zeros(B + 1, np.int32)
    mx = C.c_int32(0)
    p64 = lambda a: a.ctypes.data_as(C.POINTER(C.c_int64))
    L.check(L.lib().pa_pack_step(B, *[p64(a) for a in arrs], block_size, _p32(past), _p32(sb), _p32(bib), C.byref(mx)), None)
    return past, sb, bib, mx.value
