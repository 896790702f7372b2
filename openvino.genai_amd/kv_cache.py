"""KV cache tensors ``key_cache.<L>`` / ``value_cache.<L>`` of shape [num_blocks, Hkv, block_size, row].

Mirrors KVCacheManager (src/cpp/src/continuous_batching/cache/kv_cache_manager.hpp:56-335): growth keeps the
existing blocks, ``copy_blocks`` is the copy-on-write primitive.
"""
import ctypes as C

import numpy as np

from . import _lib as L
from .paged_attention import dtype_code, row_bytes


class KVCacheManager:
    def __init__(self, num_layers, num_kv_heads, head_size, block_size=32, kv_cache_dtype="u8", device=0, layers=None):
        """``layers``: instead of one shape for all, per layer ``((kv heads, block size, head size, type) of the key
        cache, the same of the value cache)`` -- what the reference reads off every ``key_cache.<L>`` / ``value_cache.<L>``
        input (kv_cache_manager.hpp:74-92)."""
        cfg = L.pa_config()
        cfg.device, cfg.num_heads, cfg.num_kv_heads, cfg.head_size = device, num_kv_heads, num_kv_heads, head_size
        cfg.block_size, cfg.query_dtype, cfg.kv_cache_dtype, cfg.num_layers = block_size, L.PA_F16, dtype_code(kv_cache_dtype), num_layers
        self.cfg = cfg
        self.row_bytes = row_bytes(head_size, kv_cache_dtype)
        h = C.c_void_p()
        if layers is None:
            L.check(L.lib().pa_kv_cache_create(C.byref(cfg), C.byref(h)), None)
        else:
            assert len(layers) == num_layers
            descs = (L.pa_kv_layer_desc * num_layers)()
            for d, (k, v) in zip(descs, layers):
                d.key = L.pa_kv_tensor_desc(k[0], k[1], k[2], dtype_code(k[3]))
                d.value = L.pa_kv_tensor_desc(v[0], v[1], v[2], dtype_code(v[3]))
            L.check(L.lib().pa_kv_cache_create_layers(device, None, descs, num_layers, C.byref(h)), None)
        self._h = h

    def __del__(self):
        if getattr(self, "_h", None) and L is not None:  # module globals are gone at interpreter exit
            L.lib().pa_kv_cache_destroy(self._h)
            self._h = None

    def _ck(self, status):
        L.check(status, L.lib().pa_kv_cache_last_error, self._h)

    def get_num_layers(self):
        return self.cfg.num_layers

    def get_block_size(self):
        return self.cfg.block_size

    def get_block_size_in_bytes(self):
        return int(L.lib().pa_kv_cache_block_bytes(self._h))

    def get_num_allocated_kv_blocks(self):
        return int(L.lib().pa_kv_cache_num_blocks(self._h))

    def allocate_cache_if_needed(self, num_kv_blocks):
        self._ck(L.lib().pa_kv_cache_allocate(self._h, num_kv_blocks))

    def _ptrs(self, layer):
        k, v = C.c_void_p(), C.c_void_p()
        self._ck(L.lib().pa_kv_cache_get(self._h, layer, C.byref(k), C.byref(v)))
        return k.value, v.value

    def get_key_cache(self, layer):
        return self._ptrs(layer)[0]

    def get_value_cache(self, layer):
        return self._ptrs(layer)[1]

    def copy_blocks(self, block_copy_map):
        """``{src_block: [dst_block, ...]}`` as in the reference."""
        src, dst = [], []
        for s, ds in block_copy_map.items():
            for d in ds:
                src.append(s)
                dst.append(d)
        s, d = np.ascontiguousarray(src, np.int32), np.ascontiguousarray(dst, np.int32)
        self._ck(L.lib().pa_kv_cache_copy_blocks(self._h, s.ctypes.data_as(C.POINTER(C.c_int32)),
                                                 d.ctypes.data_as(C.POINTER(C.c_int32)), len(s)))


def normalize_num_kv_blocks(num_kv_blocks, cache_size, block_size, block_bytes_all_layers, total_memory):
    """SchedulerConfig.num_kv_blocks / cache_size (GiB) -> blocks, as CacheOrchestrator::normalize_block_counts."""
    out = C.c_uint64(0)
    L.check(L.lib().pa_normalize_num_kv_blocks(num_kv_blocks, cache_size, block_size, block_bytes_all_layers,
                                               total_memory, C.byref(out)), None)
    return out.value
