"""MI355X-native PagedAttention path with the surfaces of openvino.genai's ContinuousBatchingPipeline.

The compute lives in ``csrc/libpa_amd.so`` (HIP, gfx950) behind the C-ABI of ``include/pa_amd.h``; this package is
the thin host-side mirror of the reference's names.  Nothing here computes on the CPU.
"""
from ._lib import PA_BF16, PA_F16, PA_U8, PaError, lib  # noqa: F401
from .cache_eviction import (AdaptiveRKVBlockCalculator, AdaptiveRKVConfig, AggregationMode,  # noqa: F401
                             CacheEvictionAlgorithm, CacheEvictionConfig, CacheRotationCalculator,
                             EvictionScoreManager, Evictor, KVCrushAlgorithm, KVCrushAnchorPointMode, KVCrushConfig,
                             rotation_trig_lut, snapkv_num_token_scores_to_aggregate)
from .kv_cache import KVCacheManager, normalize_num_kv_blocks  # noqa: F401
from .paged_attention import PagedAttention, pack_step, row_bytes  # noqa: F401
from .pipeline_metrics import PipelineMetrics, PipelineMetricsTracker, used_percentage  # noqa: F401
from .scheduler_config import SchedulerConfig  # noqa: F401
from .sparse_attention import (SparseAttentionConfig, SparseAttentionMode,  # noqa: F401
                               TriShapeSparseAttentionTokenSkipper, schedule_xattention_threshold)
