"""ctypes binding of ``libpa_amd.so`` (the C-ABI declared in ``include/pa_amd.h``).

There is no CPU fallback: if the HIP library has not been built, loading raises.
"""
import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
# PA_AMD_LIBRARY names another build of the library (one with instrumentation, say); it must export the same C-ABI
SO_PATH = os.environ.get("PA_AMD_LIBRARY") or os.path.join(_HERE, "csrc", "libpa_amd.so")

PA_OK = 0
PA_F16, PA_BF16, PA_U8, PA_U4 = 0, 1, 2, 3
PA_STATIC_SCRATCH_BYTES = 40 << 20
PA_AGG_SUM, PA_AGG_NORM_SUM, PA_AGG_ADAPTIVE_RKV = 0, 1, 2
(PA_KVCRUSH_ANCHOR_RANDOM, PA_KVCRUSH_ANCHOR_ZEROS, PA_KVCRUSH_ANCHOR_ONES, PA_KVCRUSH_ANCHOR_MEAN,
 PA_KVCRUSH_ANCHOR_ALTERNATING) = range(5)

STATUS_NAMES = {0: "OK", -1: "GENERAL_ERROR", -2: "NOT_IMPLEMENTED", -4: "PARAMETER_MISMATCH", -6: "OUT_OF_BOUNDS",
                -10: "NOT_ALLOCATED", -14: "INVALID_C_PARAM", -17: "UNKNOW_EXCEPTION"}

# every symbol include/pa_amd.h declares
EXPORTS = [
    "pa_version", "pa_global_last_error", "pa_create", "pa_destroy", "pa_last_error", "pa_step_begin",
    "pa_set_block_indices", "pa_set_block_indices_layers", "pa_set_alibi_slopes", "pa_forward", "pa_kv_append", "pa_attention", "pa_attention_static", "pa_synchronize", "pa_get_num_splits", "pa_set_profiling", "pa_last_kernel_ms",
    "pa_pack_step", "pa_snapkv_num_scores", "pa_kv_cache_create", "pa_kv_cache_create_layers", "pa_kv_cache_destroy", "pa_kv_cache_last_error",
    "pa_kv_cache_block_bytes", "pa_kv_cache_allocate", "pa_kv_cache_num_blocks", "pa_kv_cache_get",
    "pa_kv_cache_copy_blocks", "pa_normalize_num_kv_blocks", "pa_evictor_create", "pa_score_manager_create",
    "pa_evictor_destroy", "pa_evictor_last_error", "pa_evictor_reset_slot", "pa_evictor_register_scores",
    "pa_evictor_evict", "pa_evictor_remove_scores", "pa_evictor_get_range",
    "pa_evictor_max_cache_size_after_eviction", "pa_evictor_get_state", "pa_evictor_block_scores",
    "pa_trishape_skipped_blocks", "pa_rotation_trig_lut", "pa_rotation_data", "pa_set_rotation_trig_lut", "pa_rotate_cache",
    "pa_adaptive_rkv_diversity", "pa_evictor_register_block_diversity", "pa_select_last_error", "pa_adaptive_rkv_diversity_block_set",
    "pa_adaptive_rkv_filtered_block_diversity", "pa_adaptive_rkv_most_diverse_blocks", "pa_kvcrush_create",
    "pa_kvcrush_destroy", "pa_kvcrush_last_error", "pa_kvcrush_create_indicators", "pa_kvcrush_create_anchor_point",
    "pa_kvcrush_hamming_distances", "pa_kvcrush_representative_blocks", "pa_kvcrush_blocks_to_retain",
    "pa_xattention_threshold", "pa_set_xattention", "pa_xattention_shape", "pa_xattention_block_sums",
    "pa_xattention_retained",
]


class PaError(RuntimeError):
    """A failed C-ABI call; ``status`` carries the ov_status_e-style code."""

    def __init__(self, status, message):
        super().__init__(f"{STATUS_NAMES.get(status, status)}: {message}")
        self.status = status


class pa_config(C.Structure):
    _fields_ = [("device", C.c_int32), ("num_heads", C.c_int32), ("num_kv_heads", C.c_int32),
                ("head_size", C.c_int32), ("block_size", C.c_int32), ("query_dtype", C.c_int32),
                ("kv_cache_dtype", C.c_int32), ("num_layers", C.c_int32), ("stream", C.c_void_p),
                ("v_head_size", C.c_int32), ("value_cache_dtype_p1", C.c_int32)]


class pa_kv_tensor_desc(C.Structure):
    _fields_ = [("num_kv_heads", C.c_int32), ("block_size", C.c_int32), ("head_size", C.c_int32), ("dtype", C.c_int32)]


class pa_kv_layer_desc(C.Structure):
    _fields_ = [("key", pa_kv_tensor_desc), ("value", pa_kv_tensor_desc)]


class pa_step_meta(C.Structure):
    _fields_ = [("num_sequences", C.c_int32), ("past_lens", C.POINTER(C.c_int32)),
                ("subsequence_begins", C.POINTER(C.c_int32)), ("block_indices_begins", C.POINTER(C.c_int32)),
                ("score_aggregation_window", C.POINTER(C.c_int32)), ("max_context_len", C.c_int32),
                ("sliding_window", C.c_int32), ("scale", C.c_float)]


class pa_layer_io(C.Structure):
    _fields_ = [("query", C.c_void_p), ("key", C.c_void_p), ("value", C.c_void_p), ("key_cache", C.c_void_p),
                ("value_cache", C.c_void_p), ("num_blocks", C.c_int64), ("out", C.c_void_p), ("scores", C.c_void_p)]


class pa_evictor_config(C.Structure):
    _fields_ = [("device", C.c_int32), ("stream", C.c_void_p), ("start_size", C.c_uint64),
                ("recent_size", C.c_uint64), ("max_cache_size", C.c_uint64), ("aggregation_mode", C.c_int32),
                ("snapkv_window_size", C.c_uint64), ("block_size", C.c_uint64), ("num_decoder_layers", C.c_uint64),
                ("max_pool_window_size", C.c_uint64), ("max_sequences", C.c_uint64), ("max_tracked_tokens", C.c_uint64),
                ("adaptive_rkv_window_size", C.c_uint64), ("adaptive_rkv_attention_mass", C.c_double),
                ("kvcrush_budget", C.c_uint64), ("kvcrush_anchor_point_mode", C.c_int32),
                ("kvcrush_rng_seed", C.c_uint64)]


_lib = None


def lib():
    """The loaded library; raises if it has not been built (``python -c 'import __graft_entry__ as g; g.build()'``)."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(SO_PATH):
        raise ImportError(f"{SO_PATH} is missing: the HIP library must be built (see __graft_entry__.build); "
                          "this package has no CPU fallback")
    L = C.CDLL(SO_PATH)
    P, i32, i64, u64, vp = C.POINTER, C.c_int32, C.c_int64, C.c_uint64, C.c_void_p
    sig = {
        "pa_version": (C.c_char_p, []),
        "pa_global_last_error": (C.c_char_p, []),
        "pa_create": (i32, [P(pa_config), P(vp)]),
        "pa_destroy": (None, [vp]),
        "pa_last_error": (C.c_char_p, [vp]),
        "pa_step_begin": (i32, [vp, P(pa_step_meta)]),
        "pa_set_block_indices": (i32, [vp, i32, P(i32), i32, i64]),
        "pa_set_block_indices_layers": (i32, [vp, i32, i32, P(P(i32)), i32, i64]),
        "pa_set_alibi_slopes": (i32, [vp, P(C.c_float), i32]),
        "pa_forward": (i32, [vp, i32, P(pa_layer_io)]),
        "pa_kv_append": (i32, [vp, i32, P(pa_layer_io)]),
        "pa_attention": (i32, [vp, i32, P(pa_layer_io)]),
        "pa_attention_static": (i32, [vp, i32, P(pa_layer_io)]),
        "pa_synchronize": (i32, [vp]),
        "pa_get_num_splits": (i32, [vp]),
        "pa_set_profiling": (i32, [vp, i32]),
        "pa_last_kernel_ms": (i32, [vp, P(C.c_float)]),
        "pa_pack_step": (i32, [i32, P(i64), P(i64), P(i64), P(i64), P(i64), i32, P(i32), P(i32), P(i32), P(i32)]),
        "pa_snapkv_num_scores": (u64, [u64, u64, u64, u64]),
        "pa_trishape_skipped_blocks": (i32, [u64] * 8 + [P(u64), P(u64)]),
        "pa_rotation_trig_lut": (i32, [i32, i32, i32, C.c_double, P(C.c_float)]),
        "pa_rotation_data": (i32, [P(i64), i32, i64, i32, i32, P(i32), P(i32), i32, P(i32)]),
        "pa_set_rotation_trig_lut": (i32, [vp, P(C.c_float), i32]),
        "pa_rotate_cache": (i32, [vp, vp, i64, P(i32), i32, P(i32), i32]),
        "pa_kv_cache_create": (i32, [P(pa_config), P(vp)]),
        "pa_kv_cache_create_layers": (i32, [i32, vp, P(pa_kv_layer_desc), i32, P(vp)]),
        "pa_kv_cache_destroy": (None, [vp]),
        "pa_kv_cache_last_error": (C.c_char_p, [vp]),
        "pa_kv_cache_block_bytes": (u64, [vp]),
        "pa_kv_cache_allocate": (i32, [vp, u64]),
        "pa_kv_cache_num_blocks": (u64, [vp]),
        "pa_kv_cache_get": (i32, [vp, i32, P(vp), P(vp)]),
        "pa_kv_cache_copy_blocks": (i32, [vp, P(i32), P(i32), i32]),
        "pa_normalize_num_kv_blocks": (i32, [u64, u64, u64, u64, u64, P(u64)]),
        "pa_evictor_create": (i32, [P(pa_evictor_config), P(vp)]),
        "pa_score_manager_create": (i32, [P(pa_evictor_config), u64, P(vp)]),
        "pa_evictor_destroy": (None, [vp]),
        "pa_evictor_last_error": (C.c_char_p, [vp]),
        "pa_evictor_reset_slot": (i32, [vp, i32]),
        "pa_evictor_register_scores": (i32, [vp, i32, P(i32), P(vp), P(i64), P(u64)]),
        "pa_evictor_evict": (i32, [vp, i32, P(i32), P(i32), P(i32), i32]),
        "pa_evictor_remove_scores": (i32, [vp, i32, i32, P(i32), i32]),
        "pa_evictor_get_range": (i32, [vp, i32, i32, P(u64), P(u64)]),
        "pa_evictor_max_cache_size_after_eviction": (u64, [vp]),
        "pa_evictor_get_state": (i32, [vp, i32, i32, P(u64), P(C.c_double), P(u64), u64]),
        "pa_evictor_block_scores": (i32, [vp, i32, i32, P(C.c_double), u64, P(u64)]),
        "pa_adaptive_rkv_diversity": (i32, [vp, i32, vp, i64, i32, P(i32), vp, i64, P(i64)]),
        "pa_evictor_register_block_diversity": (i32, [vp, i32, P(i32), P(vp), P(i64)]),
        "pa_select_last_error": (C.c_char_p, []),
        "pa_adaptive_rkv_diversity_block_set": (i32, [C.c_double, u64, P(C.c_double), u64, P(u64), P(u64), P(u64)]),
        "pa_adaptive_rkv_filtered_block_diversity": (i32, [u64, P(C.c_double), u64, u64, P(u64), u64, P(C.c_double)]),
        "pa_adaptive_rkv_most_diverse_blocks": (i32, [u64, P(u64), u64, P(C.c_double), u64, P(u64), P(u64)]),
        "pa_kvcrush_create": (i32, [u64, i32, u64, u64, P(vp)]),
        "pa_kvcrush_destroy": (None, [vp]),
        "pa_kvcrush_last_error": (C.c_char_p, [vp]),
        "pa_kvcrush_create_indicators": (i32, [vp, u64, P(C.c_double), u64, P(C.c_uint8)]),
        "pa_kvcrush_create_anchor_point": (i32, [vp, u64, P(C.c_uint8), P(C.c_uint8)]),
        "pa_kvcrush_hamming_distances": (i32, [vp, u64, P(C.c_uint8), P(C.c_uint8), P(u64)]),
        "pa_kvcrush_representative_blocks": (i32, [vp, P(u64), u64, P(u64), u64, P(u64), P(u64)]),
        "pa_kvcrush_blocks_to_retain": (i32, [vp, u64, P(u64), u64, P(C.c_double), u64, P(u64), P(u64)]),
        "pa_xattention_threshold": (C.c_float, [C.c_float, u64, u64, u64, u64, i32]),
        "pa_set_xattention": (i32, [vp, P(C.c_float), i32, i32]),
        "pa_xattention_shape": (i32, [vp, i32, P(i32), P(i32), P(i32)]),
        "pa_xattention_block_sums": (i32, [vp, i32, P(C.c_float)]),
        "pa_xattention_retained": (i32, [vp, i32, P(C.c_uint8)]),
    }
    for name in EXPORTS:
        fn = getattr(L, name)  # AttributeError here = the library does not export what the header declares
        fn.restype, fn.argtypes = sig[name]
    _lib = L
    return L


def check(status, err_fn, handle=None):
    if status != PA_OK:
        msg = err_fn(handle) if handle is not None else lib().pa_global_last_error()
        raise PaError(status, (msg or b"").decode())
