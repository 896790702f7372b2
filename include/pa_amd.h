/*
 * C-ABI of the MI355X (gfx950) PagedAttention path.
 *
 * Drop-in boundary: everything openvino.genai's ContinuousBatchingPipeline hands to
 * `ov::InferRequest::infer()` for one attention layer, plus the score/eviction consumer behind it.
 * Every entry point below names the reference interface it replaces (paths relative to the
 * reference tree).  Plain pointers and sizes only; no C++ or framework types cross this boundary.
 *
 * Conventions (after src/c/src/llm_pipeline.cpp:12-23): every call returns a status code, 0 = OK,
 * negative values carry the meaning of OpenVINO's ov_status_e; no exception crosses the ABI;
 * the message of the last failure on an object is kept by `*_last_error`.
 *
 * Pointer spaces: `*_dev` / tensors named like the op's inputs live in device memory (HBM);
 * the small int32 step arrays are HOST pointers -- they are what ModelRunner::forward fills on
 * the host each step -- and are uploaded once per step by pa_step_begin.
 *
 * Threads: the library keeps no state outside its handles.  Different handles may be used by different
 * host threads at the same time (the reference drives one pipeline per thread); the calls on ONE handle
 * must not overlap.  `pa_global_last_error` is per thread.  The one exception is pa_attention_static,
 * whose calls on one GPU share that GPU's scratch array whatever handle they are made on.
 */
#ifndef PA_AMD_H
#define PA_AMD_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* status codes: the subset of ov_status_e this path can produce */
enum {
    PA_OK = 0,
    PA_GENERAL_ERROR = -1,
    PA_NOT_IMPLEMENTED = -2,
    PA_PARAMETER_MISMATCH = -4,
    PA_OUT_OF_BOUNDS = -6,
    PA_NOT_ALLOCATED = -10,
    PA_INVALID_C_PARAM = -14,
    PA_UNKNOWN_EXCEPTION = -17
};

/* element types of the tensors the op sees.  PA_U4 (cache tensors only): 4-bit codes, two per byte */
enum { PA_F16 = 0, PA_BF16 = 1, PA_U8 = 2, PA_U4 = 3 };

/* AggregationMode, include/openvino/genai/cache_eviction.hpp:19-26 */
enum { PA_AGG_SUM = 0, PA_AGG_NORM_SUM = 1, PA_AGG_ADAPTIVE_RKV = 2 };
/* KVCrushAnchorPointMode, include/openvino/genai/cache_eviction.hpp:31-43 */
enum {
    PA_KVCRUSH_ANCHOR_RANDOM = 0,
    PA_KVCRUSH_ANCHOR_ZEROS = 1,
    PA_KVCRUSH_ANCHOR_ONES = 2,
    PA_KVCRUSH_ANCHOR_MEAN = 3,
    PA_KVCRUSH_ANCHOR_ALTERNATING = 4
};

const char* pa_version(void);
/* message of the last failed call that had no object to attach it to (create functions) */
const char* pa_global_last_error(void);

/* ------------------------------------------------------------------------------------------------
 * The op.  Replaces the PagedAttentionExtension node that ov::pass::SDPAToPagedAttention inserts
 * (src/cpp/src/continuous_batching/pipeline_impl.cpp:73-92) and that runs inside
 * m_request.infer() (src/cpp/src/continuous_batching/model_runner.hpp:950-955).
 * ---------------------------------------------------------------------------------------------- */
typedef struct pa_ctx pa_ctx;

typedef struct pa_config {
    int32_t device;          /* HIP device ordinal */
    int32_t num_heads;       /* query heads */
    int32_t num_kv_heads;    /* KV heads; num_heads must be a multiple */
    int32_t head_size;       /* elements of a query / key row: a multiple of 8 up to 512 (64, 96, 128 and 256 have tuned kernels) */
    int32_t block_size;      /* tokens per KV block: the reference fixes 32 on CPU, 16 on GPU
                                (kv_cache_manager.hpp:97-110); here a knob */
    int32_t query_dtype;     /* PA_F16 | PA_BF16: query, key, value and the output */
    int32_t kv_cache_dtype;  /* PA_U8 | PA_U4 | PA_F16 | PA_BF16: what ov::hint::kv_cache_precision resolves to
                                (src/cpp/src/utils.cpp:840-863); the key cache's type, and the value cache's unless
                                value_cache_dtype_p1 says otherwise */
    int32_t num_layers;      /* decoder layers (block tables may differ per layer with eviction) */
    void* stream;            /* hipStream_t to launch on; NULL = the device's default stream.  Everything a call
                                queues is ordered with this stream: in a mixed step over a 16-bit cache one of its
                                two kernels runs on a second stream of the context's own, forked from this stream
                                and joined back into it by events inside the call */
    /* The value side where it differs from the key side: a model's value_cache.<L> may have another head size and
     * another precision than its key_cache.<L> (the reference keeps shape and precision per tensor,
     * src/cpp/src/continuous_batching/cache/kv_cache_manager.hpp:74-92, and reads the V head size on its own,
     * :274-276).  Zero in either field = as the key side, so a zero-initialised tail keeps the old meaning.  Shapes and
     * precisions that differ from layer to layer take one pa_ctx per distinct combination (contexts are cheap; they
     * share nothing but the device). */
    int32_t v_head_size;            /* elements of a value / output row; 0 = head_size */
    int32_t value_cache_dtype_p1;   /* 0 = kv_cache_dtype, else 1 + (PA_U8 | PA_U4 | PA_F16 | PA_BF16) */
} pa_config;

/* Replaces Core::compile_model + create_infer_request for this op (pipeline_impl.cpp:182,193). */
int32_t pa_create(const pa_config* cfg, pa_ctx** out);
void pa_destroy(pa_ctx* ctx);
const char* pa_last_error(const pa_ctx* ctx);

/* The per-step inputs ModelRunner::forward packs (model_runner.hpp:505-522, 802-853):
 * `past_lens` i32[B], `subsequence_begins` i32[B+1], `block_indices_begins` i32[B+1],
 * `max_context_len` i32 scalar, `score_aggregation_window` i32[B] (NULL = 1 for every sequence).
 * `scale` and `sliding_window` are graph constants in the reference; scale 0 means 1/sqrt(head_size),
 * sliding_window 0 means none. */
typedef struct pa_step_meta {
    int32_t num_sequences;
    const int32_t* past_lens;
    const int32_t* subsequence_begins;
    const int32_t* block_indices_begins;
    const int32_t* score_aggregation_window;
    int32_t max_context_len;
    int32_t sliding_window;
    float scale;
} pa_step_meta;

/* Replaces the set_tensor calls at the end of ModelRunner::forward (model_runner.hpp:907-948). */
int32_t pa_step_begin(pa_ctx* ctx, const pa_step_meta* meta);

/* `block_indices` (layer = -1: one table for all layers) or `block_indices.<layer>`
 * (model_runner.hpp:1420-1481).  Every id is checked against [0, num_blocks). */
int32_t pa_set_block_indices(pa_ctx* ctx, int32_t layer, const int32_t* block_indices, int32_t count,
                             int64_t num_blocks);
/* The `block_indices.<L>` inputs of several layers in one call (the loop over the decoder layers at
 * model_runner.hpp:1420-1481): layers first_layer .. first_layer + num_layers - 1, `block_indices_per_layer` a host
 * array of num_layers host pointers to `count` ids each.  Same checks and effect as one pa_set_block_indices per
 * layer; the ids of every layer are checked before any table changes, the tables are staged by a few host threads
 * and go up in one copy (32 tables of 65792 ids: 0.2 ms of host time, against 0.8 ms as 32 calls). */
int32_t pa_set_block_indices_layers(pa_ctx* ctx, int32_t first_layer, int32_t num_layers,
                                    const int32_t* const* block_indices_per_layer, int32_t count, int64_t num_blocks);

/* Tensors of one layer's call, all in device memory (D = head_size, Dv = the value head size):
 *   query [T, Hq*D], key [T, Hkv*D], value [T, Hkv*Dv] in query_dtype;
 *   key_cache [num_blocks, Hkv, block_size, row of D elements], value_cache [.., row of Dv elements], each in its
 *   cache type: a row of n elements is n 16-bit values for f16 / bf16, `f32 scale | f32 zero-point | n codes`
 *   (n + 8 bytes) for u8 and `f32 scale | f32 zero-point | n / 2 bytes` (element 2 i in the high nibble of byte i)
 *   for u4 (`key_cache.<L>` / `value_cache.<L>`, kv_cache_manager.hpp:30-33; the u4 row format is this library's
 *   reading of the plugin's, which the reference tree does not hold);
 *   out [T, Hq*Dv] in query_dtype; scores f32 [sum_b(past_b + new_b)] or NULL (`scores.<L>`,
 *   model_runner.hpp:23-27, 1518-1568).
 * Every tensor starts at a multiple of 16 bytes (scores: of 4); other pointers return PA_INVALID_C_PARAM. */
typedef struct pa_layer_io {
    const void* query;
    const void* key;
    const void* value;
    void* key_cache;
    void* value_cache;
    int64_t num_blocks;
    void* out;
    float* scores;
} pa_layer_io;

/* One layer's PagedAttention: KV append (+ u8 / u4 quantisation), attention, optional scores.  Tuned
 * kernels serve block_size 16, 32, 64, 128 and 256 with head size 64 or 128, K and V alike, over a u8 cache or an f16 /
 * bf16 cache of the query's type; every other combination pa_create accepts (other head sizes, a value head size or
 * value precision of its own, u4 rows, a 16-bit cache of the other 16-bit type, other block sizes) runs on shape-generic
 * kernels, correct but far from the tuned ones' speed.  In a step whose sequences all schedule one token, over a cache
 * the tuned kernels serve, the append is done by the attention kernel itself (the cache rows are the ones pa_kv_append
 * writes).  Head sizes 96 and 256 (K and V alike, the same caches) run on instantiations of the same kernels with
 * these limits: the matrix kernel keeps to 16 query rows per wave, block-sparse prefill is not offered at 96, the u8 decode
 * kernel does not take head size 256 with 16-token blocks (such steps run on the shape-generic kernel). */
int32_t pa_forward(pa_ctx* ctx, int32_t layer, const pa_layer_io* io);
/* The op's `alibi_slopes` input (input 11: f32 [num_heads]; a graph constant that SDPAToPagedAttention leaves empty
 * for models without ALiBi, and that the reference never sets itself): with slopes set, every logit gets
 * slope[head] * (key position - query position) added after the scaling.  `slopes` is a host array of `count` =
 * num_heads values; count 0 (or all zeros) takes the term away again.  A model constant: set it once after pa_create
 * (a step that has begun must begin again after a change).  The tuned kernels have no such term: a context with
 * slopes runs on the shape-generic kernels, block-sparse prefill is refused.  Parity with the plugin's term is
 * unpinned (it is applied inside the op; this is the formula of the ALiBi paper). */
int32_t pa_set_alibi_slopes(pa_ctx* ctx, const float* slopes, int32_t count);

/* The two halves of pa_forward on their own (same arguments; pa_kv_append ignores query/out/scores,
 * pa_attention ignores key/value). */
int32_t pa_kv_append(pa_ctx* ctx, int32_t layer, const pa_layer_io* io);
int32_t pa_attention(pa_ctx* ctx, int32_t layer, const pa_layer_io* io);
/* pa_attention for callers that cannot allocate (code under HIP graph capture, tight serving loops, harnesses that
 * forbid hipMalloc).  It has no counterpart in the reference.  Same arguments and results as pa_attention, for steps
 * in which every sequence schedules one token, over a u8 cache or a 16-bit cache of the query's type (block size 16 to
 * 256, a power of two; head size 64, 96, 128 or 256 -- over u8 with 16-token blocks not 256 --, K and V alike; at most
 * 16 query heads per kv head); other steps return
 * PA_NOT_IMPLEMENTED.  The split partials,
 * final maxima / denominators and the score staging live in a fixed device array of PA_STATIC_SCRATCH_BYTES bytes
 * (40 MiB; one per GPU, held until the process ends) instead of the context's growable buffers: the call itself calls
 * no hipMalloc / hipFree, and the device code of its kernels is uploaded by pa_create, not by the first call (the
 * runtime would otherwise allocate for it inside that call); a step that needs more returns PA_OUT_OF_BOUNDS and a
 * message with the byte count.  (The
 * step arrays and block tables are uploaded -- and their buffers grown -- by pa_step_begin / pa_set_block_indices,
 * as for pa_attention.)  Every call on a GPU shares that GPU's array: calls that overlap on one GPU race, also from
 * different contexts; calls in stream order on one stream do not.  Nothing in it needs clearing between calls: each
 * call writes every element it later reads. */
#define PA_STATIC_SCRATCH_BYTES (40u << 20)
int32_t pa_attention_static(pa_ctx* ctx, int32_t layer, const pa_layer_io* io);
/* Blocks until everything launched on the context's stream has finished. */
int32_t pa_synchronize(pa_ctx* ctx);
/* Number of split-K partitions of the last attention call (diagnostics). */
int32_t pa_get_num_splits(const pa_ctx* ctx);
/* Per-op timing.  The reference times the whole infer() with a host timer (ManualTimer, model_runner.hpp:951-954)
 * and has no per-op figure; here, when enabled, the dominant attention kernel of each pa_attention / pa_forward call
 * is bracketed by HIP events on the context's stream.  pa_last_kernel_ms waits for that kernel and returns its
 * duration in milliseconds. */
int32_t pa_set_profiling(pa_ctx* ctx, int32_t enable);
int32_t pa_last_kernel_ms(pa_ctx* ctx, float* ms);

/* ------------------------------------------------------------------------------------------------
 * Step packing.  Replaces the integer part of ModelRunner::forward (model_runner.hpp:802-822) and
 * SequenceGroup::get_context_len (src/cpp/src/sequence_group.hpp:744-746).
 * Per sequence: processed tokens, evicted tokens, skipped (sparse) blocks, scheduled tokens,
 * logical blocks in its table.  Outputs are the arrays of pa_step_meta.
 * ---------------------------------------------------------------------------------------------- */
int32_t pa_pack_step(int32_t num_sequences, const int64_t* processed, const int64_t* evicted,
                     const int64_t* skipped_blocks, const int64_t* scheduled, const int64_t* num_blocks,
                     int32_t block_size, int32_t* past_lens, int32_t* subsequence_begins,
                     int32_t* block_indices_begins, int32_t* max_context_len);

/* ------------------------------------------------------------------------------------------------
 * Cache rotation (used with CacheEvictionConfig::apply_rotation): after an eviction the K rows of the
 * blocks behind the evicted ones are re-rotated so that their rotary position matches their new place.
 * ---------------------------------------------------------------------------------------------- */
/* The table the pipeline builds in _prepare_rotation_data_storage
 * (src/cpp/src/continuous_batching/pipeline_impl.cpp:256-290) from CacheRotationCalculator's tables
 * (src/cpp/src/continuous_batching/cache/cache_eviction.cpp:543-575): lut[max_blocks][head_size], row i =
 * head_size/2 cosines then head_size/2 negated sines of i * block_size * rope_theta^(-2j/head_size). */
int32_t pa_rotation_trig_lut(int32_t block_size, int32_t max_blocks, int32_t head_size, double rope_theta,
                             float* lut);
/* CacheRotationCalculator::get_rotation_data (cache_eviction.cpp:577-636): for the logical blocks evicted from a
 * sequence that held num_blocks_before blocks, the kept blocks that move, in ascending order: their logical index
 * after the eviction and their delta in tokens (a multiple of block_size; delta / block_size is the table row).
 * *count receives the number of moved blocks (entries beyond `capacity` are not written).  max_blocks is the
 * table's row count (a delta of more than max_blocks blocks is an error, as in the reference). */
int32_t pa_rotation_data(const int64_t* evicted_logical_blocks, int32_t num_evicted, int64_t num_blocks_before,
                         int32_t block_size, int32_t max_blocks, int32_t* logical_block_idx,
                         int32_t* rotation_delta_tokens, int32_t capacity, int32_t* count);
/* ModelRunner::set_cache_rotation_trig_lut (src/cpp/src/continuous_batching/model_runner.hpp:1483-1509 binds it as
 * the model input `model_rotation_trig_lut`): uploads the table, [rows, head_size] floats on the host. */
int32_t pa_set_rotation_trig_lut(pa_ctx* ctx, const float* lut, int32_t rows);
/* What the op does with `rotated_block_indices.<L>` / `rotation_deltas.<L>` before attention
 * (model_runner.hpp:1483-1509; deltas filled at pipeline_impl.cpp:856-872): re-rotates, in place, every K row of the
 * listed physical blocks of one layer's key cache (device pointer).  rotated_block_indices [n] and rotation_deltas
 * [n, deltas_per_block] (table rows; deltas_per_block is 1 or block_size) are host arrays.  Key caches of u8, f16
 * or bf16 rows; u4 rows return PA_NOT_IMPLEMENTED. */
int32_t pa_rotate_cache(pa_ctx* ctx, void* key_cache, int64_t num_blocks, const int32_t* rotated_block_indices,
                        int32_t num_rotated, const int32_t* rotation_deltas, int32_t deltas_per_block);

/* TriShapeSparseAttentionTokenSkipper::get_skipped_blocks
 * (src/cpp/src/continuous_batching/sparse_attention.cpp:12-35, constructor checks sparse_attention.hpp:36-49): the
 * logical blocks left out of a sequence's block table for the next prefill chunk are
 * [*first_skipped, *first_skipped + *num_skipped).  num_cached_tokens = processed - evicted tokens
 * (src/cpp/src/sequence_group.hpp:858-861).  The attention kernels need nothing more: they walk whatever table
 * pa_set_block_indices receives, and pa_pack_step subtracts the skipped blocks from past_lens. */
int32_t pa_trishape_skipped_blocks(uint64_t block_size, uint64_t num_last_dense_tokens_in_prefill,
                                   uint64_t num_retained_start_tokens_in_cache,
                                   uint64_t num_retained_recent_tokens_in_cache, uint64_t prompt_len,
                                   uint64_t num_processed_tokens, uint64_t num_scheduled_tokens,
                                   uint64_t num_cached_tokens, uint64_t* first_skipped, uint64_t* num_skipped);

/* ------------------------------------------------------------------------------------------------
 * Block-sparse prefill (SparseAttentionMode::XATTENTION, include/openvino/genai/sparse_attention.hpp:17-20,67-83).
 * The estimate and the selection run inside the op in the reference (OpenVINO Runtime); what the reference tree holds
 * is the inputs it sets and their description (site/docs/concepts/optimization-techniques/
 * sparse-attention-prefill.md:48-69).
 * ---------------------------------------------------------------------------------------------- */
/* Scheduler::_schedule_xattention_threshold (src/cpp/src/continuous_batching/scheduler.hpp:922-940) for a pipeline
 * that runs in XATTENTION mode: the threshold a sequence group gets for the coming step -- 0 (dense) in the
 * generation phase and for a chunk that ends fewer than num_last_dense_tokens_in_prefill tokens before the
 * prompt's end, else the configured one.  can_generate_tokens: SequenceGroup::can_generate_tokens()
 * (src/cpp/src/sequence_group.hpp:578-580). */
float pa_xattention_threshold(float configured_threshold, uint64_t num_last_dense_tokens_in_prefill, uint64_t prompt_len,
                              uint64_t num_processed_tokens, uint64_t num_scheduled_tokens, int32_t can_generate_tokens);
/* ModelRunner::_set_xattention_tensors (src/cpp/src/continuous_batching/model_runner.hpp:1623-1656): the inputs
 * `xattention_threshold.<L>` (f32 [B], host array here; the reference binds one tensor to every layer),
 * `xattention_block_size` and `xattention_stride`.  Call after pa_step_begin and before the step's pa_forward /
 * pa_attention calls; pa_step_begin forgets it again.  thresholds NULL or all zero = dense.  A sequence with a
 * threshold above zero that schedules more than one token is attended block-sparsely:
 *   - positions are absolute: block I covers [I * block_size, (I + 1) * block_size), strided group i covers
 *     [i * stride, (i + 1) * stride);
 *   - importance of strided groups (i, j <= i): softmax over j of
 *         scale / stride * sum_{s < stride} q[i * stride + stride-1-s] . k[j * stride + s]
 *     (the antidiagonals of the stride x stride tiles of Q K^T); importance of a block pair (I, J) = the sum over
 *     its groups; tokens outside the chunk count as zero vectors;
 *   - per (query head, I): key blocks 0 and I are kept, then the others in descending importance until the kept sum
 *     reaches threshold * the row's sum; a query row then sees a key position only if its block pair was kept.
 * Needs a cache block_size of 32, 64, 128 or 256, head_size 64 / 128 / 256 (K and V alike), a u8 cache or one of the query's
 * type; xattention_block_size a power of two >= 32, xattention_stride a power of two <= 32 (PA_NOT_IMPLEMENTED
 * otherwise). */
int32_t pa_set_xattention(pa_ctx* ctx, const float* thresholds, int32_t xattention_block_size,
                          int32_t xattention_stride);
/* Diagnostics of the last pa_attention / pa_forward call of the step (no counterpart in the reference, whose op keeps
 * the selection to itself).  For one sequence of the step: the first query block its chunk touches, the number of
 * query blocks and of key blocks (all 0 for a dense sequence); the block importances and the kept pairs as host
 * arrays [num_heads][num_query_blocks][num_key_blocks] (the calls wait for the context's stream). */
int32_t pa_xattention_shape(const pa_ctx* ctx, int32_t sequence, int32_t* first_query_block, int32_t* num_query_blocks,
                            int32_t* num_key_blocks);
int32_t pa_xattention_block_sums(pa_ctx* ctx, int32_t sequence, float* sums);
int32_t pa_xattention_retained(pa_ctx* ctx, int32_t sequence, uint8_t* retained);

/* SnapKVScoreAggregationCalculator::get_num_token_scores_to_aggregate
 * (src/cpp/src/continuous_batching/cache/cache_eviction.cpp:638-657). */
uint64_t pa_snapkv_num_scores(uint64_t snapkv_window_size, uint64_t prompt_len, uint64_t num_scheduled_tokens,
                              uint64_t num_processed_tokens);

/* ------------------------------------------------------------------------------------------------
 * KV cache tensors.  Replaces KVCacheManager (src/cpp/src/continuous_batching/cache/
 * kv_cache_manager.hpp:56-335) and CacheOrchestrator::normalize_block_counts
 * (cache_orchestrator.hpp:781-869) for the KV-only case.
 * ---------------------------------------------------------------------------------------------- */
typedef struct pa_kv_cache pa_kv_cache;

/* One cache tensor as the reference reads it off the model's `key_cache.<L>` / `value_cache.<L>` input: shape
 * [num_blocks, num_kv_heads, block_size, head_size] and element type (kv_cache_manager.hpp:74-92).  Any PA_* cache
 * type; sub-byte types halve the bytes (kv_cache_manager.hpp:152-157). */
typedef struct pa_kv_tensor_desc {
    int32_t num_kv_heads;
    int32_t block_size;
    int32_t head_size;
    int32_t dtype;
} pa_kv_tensor_desc;
typedef struct pa_kv_layer_desc {
    pa_kv_tensor_desc key, value;
} pa_kv_layer_desc;

/* every layer alike, from the op's configuration (value side included) */
int32_t pa_kv_cache_create(const pa_config* cfg, pa_kv_cache** out);
/* shape and precision per layer and per tensor (m_key_shapes / m_value_shapes / m_key_precisions /
 * m_value_precisions, kv_cache_manager.hpp:74-92) */
int32_t pa_kv_cache_create_layers(int32_t device, void* stream, const pa_kv_layer_desc* layers, int32_t num_layers,
                                  pa_kv_cache** out);
void pa_kv_cache_destroy(pa_kv_cache* cache);
const char* pa_kv_cache_last_error(const pa_kv_cache* cache);
/* bytes of one block over all layers, K and V (get_block_size_in_bytes) */
uint64_t pa_kv_cache_block_bytes(const pa_kv_cache* cache);
/* allocate_cache_if_needed: grows every layer to num_kv_blocks, keeping blocks [0, old) */
int32_t pa_kv_cache_allocate(pa_kv_cache* cache, uint64_t num_kv_blocks);
uint64_t pa_kv_cache_num_blocks(const pa_kv_cache* cache);
/* get_key_cache / get_value_cache: device pointers of one layer */
int32_t pa_kv_cache_get(const pa_kv_cache* cache, int32_t layer, void** key_cache, void** value_cache);
/* copy_blocks (copy-on-write): block src[i] -> dst[i] in every layer */
int32_t pa_kv_cache_copy_blocks(pa_kv_cache* cache, const int32_t* src, const int32_t* dst, int32_t count);
/* SchedulerConfig.num_kv_blocks / cache_size (GiB) -> blocks to allocate; 0 = grow on demand
 * (include/openvino/genai/scheduler_config.hpp:25-31). */
int32_t pa_normalize_num_kv_blocks(uint64_t num_kv_blocks, uint64_t cache_size_gib, uint64_t block_size,
                                   uint64_t block_bytes_all_layers, uint64_t total_memory, uint64_t* out);

/* ------------------------------------------------------------------------------------------------
 * Score accumulation and eviction.  Replaces EvictionScoreManager and CacheEvictionAlgorithm
 * (src/cpp/src/continuous_batching/cache/cache_eviction.hpp:23-248, cache_eviction.cpp:9-524) as
 * driven by ContinuousBatchingImpl::_maybe_evict_cache_blocks (pipeline_impl.cpp:884-959).
 * State (f64 scores, u64 lifetime counters) stays in device memory, one slot per tracked sequence;
 * the per-token scores are read straight from the `scores.<L>` device buffers the op wrote.
 * SUM, NORM_SUM and ADAPTIVE_RKV are implemented, KVCrush included; sparse-prefill skip sets must
 * be empty (the reference registers no scores for steps with skipped blocks,
 * pipeline_impl.cpp:909-912).  The choice among blocks that ADAPTIVE_RKV and KVCrush make runs on
 * the host over the block scores (a few hundred values per sequence and layer), with the standard
 * library facilities the reference uses, so that ties fall the same way.
 * ---------------------------------------------------------------------------------------------- */
typedef struct pa_evictor pa_evictor;

typedef struct pa_evictor_config {
    int32_t device;
    void* stream;                   /* NULL = default stream */
    uint64_t start_size;            /* CacheEvictionConfig (cache_eviction.hpp:110-226) */
    uint64_t recent_size;
    uint64_t max_cache_size;
    int32_t aggregation_mode;       /* PA_AGG_SUM | PA_AGG_NORM_SUM | PA_AGG_ADAPTIVE_RKV */
    uint64_t snapkv_window_size;
    uint64_t block_size;
    uint64_t num_decoder_layers;
    uint64_t max_pool_window_size;  /* 7 in the pipeline (pipeline_impl.cpp:900) */
    uint64_t max_sequences;         /* slots */
    uint64_t max_tracked_tokens;    /* capacity per slot and layer */
    /* AdaptiveRKVConfig (include/openvino/genai/cache_eviction.hpp:93-100); read in ADAPTIVE_RKV mode only */
    uint64_t adaptive_rkv_window_size;     /* 1..32; the reference's default is 8 */
    double adaptive_rkv_attention_mass;    /* the reference's default is 0.9 */
    /* KVCrushConfig (include/openvino/genai/cache_eviction.hpp:48-91); budget 0 switches KVCrush off */
    uint64_t kvcrush_budget;
    int32_t kvcrush_anchor_point_mode;     /* PA_KVCRUSH_ANCHOR_* */
    uint64_t kvcrush_rng_seed;
} pa_evictor_config;

/* CacheEvictionConfig ctor + CacheEvictionAlgorithm ctor checks (cache_eviction.hpp:130-136,
 * cache_eviction.cpp:288-294). */
int32_t pa_evictor_create(const pa_evictor_config* cfg, pa_evictor** out);
/* Bare EvictionScoreManager: no areas, `ignore_first_n_blocks` given directly (cache_eviction.hpp:47). */
int32_t pa_score_manager_create(const pa_evictor_config* cfg, uint64_t ignore_first_n_blocks, pa_evictor** out);
void pa_evictor_destroy(pa_evictor* ev);
const char* pa_evictor_last_error(const pa_evictor* ev);
/* forget a slot's state (sequence finished) */
int32_t pa_evictor_reset_slot(pa_evictor* ev, int32_t slot);

/* register_new_token_scores for a batch of sequences: `scores_per_layer` is a host array of
 * num_decoder_layers device pointers (`scores.<L>`); sequence i's vector is
 * [offsets[i], offsets[i+1]) in each of them; num_snapkv_scores may be NULL (all 0).
 * The call returns once its kernel is QUEUED on the evictor's stream: the host arrays are free again, the
 * `scores.<L>` device tensors are read later, in stream order.  Work that follows on the same stream (the next
 * step's pa_forward rewriting the tensors, pa_evictor_evict, ...) is ordered behind that read by the stream
 * itself; rewriting the tensors from ANOTHER stream needs an event or a synchronisation in between, and so does
 * producing them on another stream than the evictor's (give the evictor the pa_ctx's stream).  Of the pair
 * register / evict, register returns with its work in flight, pa_evictor_evict returns synchronised (its lists are
 * host arrays). */
int32_t pa_evictor_register_scores(pa_evictor* ev, int32_t num_sequences, const int32_t* slots,
                                   const float* const* scores_per_layer, const int64_t* offsets,
                                   const uint64_t* num_snapkv_scores);
/* register_block_diversity (cache_eviction.cpp:526-541) for a batch of sequences, ADAPTIVE_RKV mode:
 * `diversity_per_layer` is a host array of num_decoder_layers device pointers
 * (`adaptive_rkv_diversity.<L>`); sequence i's [evictable / block_size, evictable] f32 matrix is
 * [offsets[i], offsets[i+1]) in each of them.  The values are copied (one launch for the whole batch, queued on
 * the evictor's stream like pa_evictor_register_scores: the tensors are read in stream order, the host arrays are
 * free on return); they are dropped by the next pa_evictor_evict that names the sequence. */
int32_t pa_evictor_register_block_diversity(pa_evictor* ev, int32_t num_sequences, const int32_t* slots,
                                            const float* const* diversity_per_layer, const int64_t* offsets);
/* evict_logical_blocks for a batch of sequences.  counts[i*L + l] = blocks evicted for sequence i,
 * layer l; their logical indices (ascending, start area included) are written to
 * blocks[(i*L + l)*max_blocks_per_entry ...].  State of the evicted blocks is dropped. */
int32_t pa_evictor_evict(pa_evictor* ev, int32_t num_sequences, const int32_t* slots, int32_t* counts,
                         int32_t* blocks, int32_t max_blocks_per_entry);
/* EvictionScoreManager::remove_scores: `blocks` index the tracked area, ascending */
int32_t pa_evictor_remove_scores(pa_evictor* ev, int32_t slot, int32_t layer, const int32_t* blocks, int32_t count);
/* get_evictable_block_range; (0, 0) when no eviction is due */
int32_t pa_evictor_get_range(const pa_evictor* ev, int32_t slot, int32_t layer, uint64_t* begin, uint64_t* end);
uint64_t pa_evictor_max_cache_size_after_eviction(const pa_evictor* ev);
/* tracked length, and copies of the device state to host (either pointer may be NULL) */
int32_t pa_evictor_get_state(pa_evictor* ev, int32_t slot, int32_t layer, uint64_t* length, double* scores,
                             uint64_t* counters, uint64_t capacity);
/* importances of the blocks in the evictable range (get_scores_for_all_evictable_blocks) */
int32_t pa_evictor_block_scores(pa_evictor* ev, int32_t slot, int32_t layer, double* out, uint64_t capacity,
                                uint64_t* count);

/* The op's `adaptive_rkv_diversity.<L>` output for one layer (requested through the inputs
 * `adaptive_rkv_start_size` / `adaptive_rkv_evictable_sizes`, model_runner.hpp:1658-1690; read back
 * at model_runner.hpp:1570-1621).  For every sequence b of the current step with
 * evictable_sizes[b] > 0, in step order: a [evictable_sizes[b] / block_size, evictable_sizes[b]]
 * f32 matrix over the keys at positions [start_size, start_size + evictable_sizes[b]) -- minus the
 * sum, over the rows of a block, of the head-averaged cosine similarities that are not below their
 * row's mean.  The matrices are concatenated in `diversity` (device, `capacity` floats);
 * offsets[b] .. offsets[b+1] (host, B + 1 entries, may be NULL) is sequence b's span.  Uses the
 * block table of `layer` set by pa_set_block_indices in this step.  Block size 32 with head size 64, 96, 128 or 256
 * over u8 / f16 / bf16 keys runs on the matrix cores, every other shape pa_create accepts on the vector unit (the
 * same values, far slower).  `evictable_sizes` is a HOST array of B entries.  The optional block-set inputs
 * (`adaptive_rkv_diversity_block_set_indices.<L>`, model_runner.hpp:1691-1770) only permit computing
 * less; every block is computed here.
 * The arithmetic of this output lives in OpenVINO (2026.4 development line, the reference's pinned
 * dependency), not in the reference tree: see the note on parity in the kernel's source. */
int32_t pa_adaptive_rkv_diversity(pa_ctx* ctx, int32_t layer, const void* key_cache, int64_t num_blocks,
                                  int32_t start_size, const int32_t* evictable_sizes, float* diversity,
                                  int64_t capacity, int64_t* offsets);

/* ------------------------------------------------------------------------------------------------
 * Block selection helpers of the eviction step, host only (no device work).  The evictor above calls
 * them itself; they are exported because the reference exposes them as classes with tests of their
 * own.
 * ---------------------------------------------------------------------------------------------- */
const char* pa_select_last_error(void);
/* AdaptiveRKVBlockCalculator::get_diversity_block_set (cache_eviction.cpp:659-692): `set_out` has
 * room for num_blocks indices (ascending); *num_blocks_kept = blocks kept for their attention mass. */
int32_t pa_adaptive_rkv_diversity_block_set(double attention_mass, uint64_t max_num_blocks_kept,
                                            const double* block_scores, uint64_t num_blocks, uint64_t* set_out,
                                            uint64_t* set_count, uint64_t* num_blocks_kept);
/* AdaptiveRKVBlockCalculator::get_filtered_block_diversity (cache_eviction.cpp:694-713): `out` has
 * eviction_size / block_size entries. */
int32_t pa_adaptive_rkv_filtered_block_diversity(uint64_t block_size, const double* unfiltered, uint64_t num_values,
                                                 uint64_t eviction_size, const uint64_t* set, uint64_t set_count,
                                                 double* out);
/* AdaptiveRKVBlockCalculator::get_most_diverse_blocks (cache_eviction.cpp:716-737) */
int32_t pa_adaptive_rkv_most_diverse_blocks(uint64_t num_blocks_left_to_fill, const uint64_t* set, uint64_t set_count,
                                            const double* filtered, uint64_t num_filtered, uint64_t* out,
                                            uint64_t* out_count);

/* KVCrushAlgorithm (src/cpp/src/continuous_batching/cache/kvcrush.hpp:17-60, kvcrush.cpp:9-174).
 * Indicator and anchor vectors are one byte (0 / 1) per token / in-block position. */
typedef struct pa_kvcrush pa_kvcrush;
int32_t pa_kvcrush_create(uint64_t budget, int32_t anchor_point_mode, uint64_t rng_seed, uint64_t block_size,
                          pa_kvcrush** out);
void pa_kvcrush_destroy(pa_kvcrush* k);
const char* pa_kvcrush_last_error(const pa_kvcrush* k);
/* create_indicators_kvcrush (kvcrush.cpp:15-36) */
int32_t pa_kvcrush_create_indicators(pa_kvcrush* k, uint64_t num_tokens, const double* layer_scores, uint64_t num_scores,
                                     uint8_t* indicators_out);
/* create_anchor_point_kvcrush (kvcrush.cpp:38-82); `anchor_out` has block_size entries */
int32_t pa_kvcrush_create_anchor_point(pa_kvcrush* k, uint64_t num_tokens, const uint8_t* indicators, uint8_t* anchor_out);
/* calculate_hamming_distance_kvcrush (kvcrush.cpp:84-111); one distance per block */
int32_t pa_kvcrush_hamming_distances(pa_kvcrush* k, uint64_t num_tokens, const uint8_t* indicators, const uint8_t* anchor,
                                     uint64_t* distances_out);
/* get_representative_blocks_kvcrush (kvcrush.cpp:113-148); `out` has room for num_eligible indices */
int32_t pa_kvcrush_representative_blocks(pa_kvcrush* k, const uint64_t* distances, uint64_t num_blocks,
                                         const uint64_t* eligible, uint64_t num_eligible, uint64_t* out,
                                         uint64_t* out_count);
/* get_indices_of_blocks_to_retain_using_kvcrush (kvcrush.cpp:150-174) */
int32_t pa_kvcrush_blocks_to_retain(pa_kvcrush* k, uint64_t num_tokens, const uint64_t* evicted, uint64_t num_evicted,
                                    const double* layer_scores, uint64_t num_scores, uint64_t* out, uint64_t* out_count);

#ifdef __cplusplus
}
#endif
#endif /* PA_AMD_H */
