"""`PipelineMetrics` of the reference (include/openvino/genai/continuous_batching_pipeline.hpp:33-75, bound at
src/python/py_continuous_batching_pipeline.cpp:459-467) and the bookkeeping that fills the fields this path owns:
cache usage per step, its maximum and running average, and the duration of a step's forward.

The block allocator itself stays the caller's (the scheduler hands this path block tables); what it knows per step --
free blocks per layer, total blocks -- is all the usage figures need.
"""
import collections
import time

import numpy as np


class PipelineMetrics:
    """Field names and defaults of the reference's struct; `kv_cache_size_in_bytes` is its deprecated alias."""

    def __init__(self):
        self.requests = 0
        self.scheduled_requests = 0
        self.cache_usage = 0.0
        self.max_cache_usage = 0.0
        self.avg_cache_usage = 0.0
        self.inference_duration = 0.0   # microseconds, the last step's forward
        self.sampling_duration = 0.0    # microseconds; sampling is outside this path and stays 0 unless the caller sets it
        self.cache_size_in_bytes = 0

    @property
    def kv_cache_size_in_bytes(self):
        return self.cache_size_in_bytes

    def copy(self):
        m = PipelineMetrics()
        m.__dict__.update(self.__dict__)
        return m


def used_percentage(num_free_blocks_per_layer, total_num_blocks):
    """BlockAllocator::get_used_percentage (cache/block_manager.hpp:588-592): float32 arithmetic of
    (layers * total - sum of free) / (layers * total) * 100."""
    free = [int(x) for x in num_free_blocks_per_layer]
    denom = len(free) * int(total_num_blocks)
    if denom == 0:
        return float("nan")  # 0 / 0 in the reference
    return float(np.float32(denom - sum(free)) / np.float32(denom) * np.float32(100))


class PipelineMetricsTracker:
    """What ContinuousBatchingImpl::step does to m_pipeline_metrics (pipeline_impl.cpp:394-398, 426-431, 779-795)."""

    AVG_CACHE_USAGE_WINDOW_SIZE_IN_STEPS = 1000  # pipeline_impl.hpp:33

    def __init__(self):
        self._metrics = PipelineMetrics()
        self._previous = collections.deque()

    def get_metrics(self):
        return self._metrics.copy()

    def register_step(self, num_free_blocks_per_layer, total_num_blocks, requests=0, scheduled_requests=0,
                      cache_size_in_bytes=0):
        """After scheduling: the step's cache usage (scheduler.hpp:245), the maximum and the running average over at
        most 1000 steps; request counts and the cache size are passed through."""
        m = self._metrics
        usage = used_percentage(num_free_blocks_per_layer, total_num_blocks)
        m.requests, m.scheduled_requests = int(requests), int(scheduled_requests)
        m.cache_size_in_bytes = int(cache_size_in_bytes)
        m.cache_usage = usage
        m.max_cache_usage = max(m.max_cache_usage, usage)
        if len(self._previous) >= self.AVG_CACHE_USAGE_WINDOW_SIZE_IN_STEPS:
            self._previous.popleft()
        self._previous.append(usage)
        m.avg_cache_usage = float(np.float32(sum(float(x) for x in self._previous) / len(self._previous)))
        return usage

    def time_forward(self, synchronize):
        """Context manager around a step's layer calls: wall clock from entry until `synchronize()` returns (the
        reference's forward returns when infer() has finished), in microseconds, into `inference_duration`."""
        return _ForwardTimer(self._metrics, synchronize)

    def reset_cache_usage_statistics(self):
        """_reset_cache_usage_statistics (pipeline_impl.cpp:791-795), at the start of a generate() call."""
        self._previous.clear()
        self._metrics.max_cache_usage = 0.0
        self._metrics.avg_cache_usage = 0.0


class _ForwardTimer:
    def __init__(self, metrics, synchronize):
        self._m, self._sync = metrics, synchronize

    def __enter__(self):
        self._t0 = time.perf_counter()
        return self

    def __exit__(self, exc_type, exc, tb):
        if exc_type is None:
            self._sync()
            self._m.inference_duration = (time.perf_counter() - self._t0) * 1e6
        return False
