// Host side of the C-ABI: contexts, step planning, validation, KV cache tensors, step packing.
// C++ behind `extern "C"`; no exception leaves this file.
#include <algorithm>
#include <cmath>
#include <cstring>
#include <mutex>
#include <stdexcept>
#include <string>
#include <vector>

#include "../../include/pa_amd.h"
#include "pa_device.h"
#include "host_parallel.h"

namespace {

thread_local std::string g_last_error;

struct StatusError : std::runtime_error {
    int32_t code;
    StatusError(int32_t c, const std::string& m) : std::runtime_error(m), code(c) {}
};

#define PA_REQUIRE(cond, code, msg)                                   \
    do {                                                              \
        if (!(cond)) throw StatusError((code), (msg));                \
    } while (0)

#define HIP_CHECK(expr)                                                                               \
    do {                                                                                              \
        hipError_t e_ = (expr);                                                                       \
        if (e_ != hipSuccess)                                                                         \
            throw StatusError(e_ == hipErrorOutOfMemory ? PA_NOT_ALLOCATED : PA_GENERAL_ERROR,        \
                              std::string(#expr) + ": " + hipGetErrorString(e_));                     \
    } while (0)

// Device buffer that only ever grows.
struct DevBuf {
    void* p = nullptr;
    size_t cap = 0;
    void reserve(size_t bytes) {
        if (bytes <= cap) return;
        if (p) {  // work in flight may still use the old buffer
            HIP_CHECK(hipDeviceSynchronize());
            HIP_CHECK(hipFree(p));
        }
        p = nullptr;
        cap = 0;
        size_t want = std::max<size_t>(bytes, 256);
        HIP_CHECK(hipMalloc(&p, want));
        cap = want;
    }
    void release() {
        if (p) (void)hipFree(p);
        p = nullptr;
        cap = 0;
    }
    template <class T>
    T* as() const { return static_cast<T*>(p); }
};

// Pinned host memory that only ever grows (allocated, never registered): uploads from it are plain DMA, where a
// pageable source of a few hundred KB is pinned and unpinned by the runtime on every copy.
struct PinnedBuf {
    void* p = nullptr;
    size_t cap = 0;
    void reserve(size_t bytes) {
        if (bytes <= cap) return;
        if (p) HIP_CHECK(hipHostFree(p));
        p = nullptr;
        cap = 0;
        const size_t want = std::max<size_t>(bytes + bytes / 2, 4096);
        HIP_CHECK(hipHostMalloc(&p, want, hipHostMallocDefault));
        cap = want;
    }
    void release() {
        if (p) (void)hipHostFree(p);
        p = nullptr;
        cap = 0;
    }
    template <class T>
    T* as() const { return static_cast<T*>(p); }
};

void check_config(const pa_config* c) {
    PA_REQUIRE(c, PA_INVALID_C_PARAM, "config is null");
    PA_REQUIRE(c->num_heads > 0 && c->num_kv_heads > 0 && c->num_heads % c->num_kv_heads == 0, PA_PARAMETER_MISMATCH,
               "num_heads must be a positive multiple of num_kv_heads");
    auto head_ok = [](int32_t d) { return d >= 8 && d <= pa::GENERIC_MAX_HEAD_SIZE && d % 8 == 0; };
    auto cache_dt_ok = [](int32_t dt) { return dt == PA_F16 || dt == PA_BF16 || dt == PA_U8 || dt == PA_U4; };
    PA_REQUIRE(head_ok(c->head_size), PA_NOT_IMPLEMENTED, "head_size must be a multiple of 8 between 8 and 512");
    PA_REQUIRE(c->v_head_size == 0 || head_ok(c->v_head_size), PA_NOT_IMPLEMENTED,
               "v_head_size must be 0 (= head_size) or a multiple of 8 between 8 and 512");
    PA_REQUIRE(c->block_size > 0, PA_PARAMETER_MISMATCH, "block_size must be positive");
    PA_REQUIRE(c->query_dtype == PA_F16 || c->query_dtype == PA_BF16, PA_PARAMETER_MISMATCH,
               "query_dtype must be PA_F16 or PA_BF16");
    PA_REQUIRE(cache_dt_ok(c->kv_cache_dtype), PA_PARAMETER_MISMATCH, "kv_cache_dtype must be PA_U8, PA_U4, PA_F16 or PA_BF16");
    PA_REQUIRE(c->value_cache_dtype_p1 == 0 || cache_dt_ok(c->value_cache_dtype_p1 - 1), PA_PARAMETER_MISMATCH,
               "value_cache_dtype_p1 must be 0 (= kv_cache_dtype) or 1 + PA_U8 / PA_U4 / PA_F16 / PA_BF16");
    PA_REQUIRE(c->num_layers > 0, PA_PARAMETER_MISMATCH, "num_layers must be positive");
    int ndev = 0;
    HIP_CHECK(hipGetDeviceCount(&ndev));
    PA_REQUIRE(c->device >= 0 && c->device < ndev, PA_OUT_OF_BOUNDS, "no such HIP device");
}

// The value side of a configuration (0 in either field = as the key side).
int32_t v_head(const pa_config& c) { return c.v_head_size ? c.v_head_size : c.head_size; }
int32_t v_dtype(const pa_config& c) { return c.value_cache_dtype_p1 ? c.value_cache_dtype_p1 - 1 : c.kv_cache_dtype; }
// K and V alike, in a type the tuned kernels read (they also want head size 64 or 128: checked where they are chosen)
bool kv_alike(const pa_config& c) {
    return v_head(c) == c.head_size && v_dtype(c) == c.kv_cache_dtype && c.kv_cache_dtype != PA_U4;
}

// Fixed device scratch of pa_attention_static: one copy per GPU the library runs on, held until the process ends.
// In host code this name is only a handle for hipGetSymbolAddress; device code and every launch use the resolved
// pointer.
constexpr size_t STATIC_SCRATCH_BYTES = PA_STATIC_SCRATCH_BYTES;
static __device__ __align__(256) uint8_t scratch[STATIC_SCRATCH_BYTES];

constexpr int MAX_DEVICES = 64;
std::mutex g_scratch_mutex;
void* g_scratch_ptr[MAX_DEVICES] = {};

// The device address of `scratch` on `device`, which must be the current device.
void* resolve_static_scratch(int device) {
    PA_REQUIRE(device >= 0 && device < MAX_DEVICES, PA_OUT_OF_BOUNDS, "device ordinal beyond the scratch table");
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[device]) {
        void* p = nullptr;
        HIP_CHECK(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
        PA_REQUIRE(p, PA_GENERAL_ERROR, "hipGetSymbolAddress returned a null address for the static scratch");
        g_scratch_ptr[device] = p;
    }
    return g_scratch_ptr[device];
}

}  // namespace

struct pa_ctx {
    pa_config cfg{};
    hipStream_t stream = nullptr;
    std::string error;
    uint8_t* static_scratch = nullptr;  // this device's copy of the fixed scratch (pa_attention_static)
    // step state
    bool step_ready = false;
    int32_t B = 0, T = 0, max_kv = 0, total_scores = 0, total_block_ids = 0, nsplit = 1, generic_nsplit = 1;
    int32_t sliding_window = 0;
    float scale = 0.0f;
    std::vector<int32_t> h_past, h_sb, h_bib;
    DevBuf meta;  // past | sb | bib | window | score_off | token_seq
    DevBuf items;     // work items of the MFMA kernel, then the per-token split counts
    DevBuf dec_list;  // single-token sequences (for the u8 decode kernel)
    DevBuf trig_lut, rot_args;  // cache rotation: [rows, head_size] table; block ids + deltas of one call
    DevBuf div_seqs, div_stats, div_mean, div_colsum;  // block diversity: per-call sequence list and workspace
    // block-sparse prefill (XAttention) of the current step
    std::vector<pa::XattSeq> h_xseq;
    std::vector<int32_t> h_xseq_of;
    std::vector<pa::PrefillItem> h_items;
    int32_t xatt_block = 0, xatt_stride = 0;
    bool x_ran = false;               // a layer call of this step has produced block sums and masks
    int32_t n_sparse = 0, x_ntiles = 0, x_keep_words = 1, x_max_nqs = 0, x_max_nqb = 0, x_max_nkb = 0;
    size_t x_tiles_off = 0, x_seq_of_off = 0;
    DevBuf x_plan;                    // XattSeq list | tiles of the estimate | sequence -> list index
    DevBuf x_logits, x_sums, x_mask, x_item_keep;
    int32_t trig_rows = 0;
    std::vector<int32_t> h_dec;
    std::vector<int32_t> h_dec16;     // single-token sequences of a 16-bit-cache step (also listed as matrix-kernel items)
    DevBuf dec16_list;
    std::vector<int32_t> h_multi;     // sequences that schedule more than one token
    DevBuf multi_list;
    DevBuf tile_max;   // per (head, 32-token tile) maxima of single-token sequences handled by the matrix kernel
    bool dec_in_order = false, dec16_in_order = false;  // the lists hold 0 .. B-1 in order: every sequence, none moved
    bool stash_ok = false;  // the step's single-token items are short enough to keep their probabilities in LDS
    int32_t n_items = 0, n_wide = 0, max_split = 1;
    size_t tok_nsplit_off = 0;
    // single-token sequences the matrix kernel may take (16-bit caches): their work items, and behind the split
    // counts a per-sequence flag array (for the call that hands them to the decode kernel instead)
    int32_t n_single = 0;
    size_t single_idx_off = 0;
    size_t merge_tok_off = 0;         // tokens whose context was cut into several ranges, in the same upload
    int32_t n_merge = 0;
    pa::StepDev dev{};
    // block tables: shared (index 0 of `tables` when shared) or per layer
    std::vector<DevBuf> tables;
    std::vector<const void*> table_ptr;  // where each table lives: its own buffer, or a slice of table_pool
    DevBuf table_pool;                   // the tables of a whole-model call, one after the other
    std::vector<int32_t> table_count;
    std::vector<int64_t> table_bound;  // largest block id of each table + 1: the smallest cache it may be used with
    // u8 decode kernel: its split-K plan without / with scores (fixed per step) and, behind every table, the
    // per-(sequence, split) descriptors of both plans
    struct DecPlan { int32_t nsplit = 1, max_tiles = 1, waves = 4; } dec_plan[2];
    size_t desc_off[2] = {0, 0};       // byte offsets of the two descriptor arrays in a table's buffer
    // the step's host arrays (packed metadata, work items, lists, block tables with their descriptors) pass through
    // this pinned area on their way to the device: pieces are handed out front to back, their copies are queued and not
    // waited for, and pa_step_begin starts over at the front once it has waited for the stream
    PinnedBuf step_staging;
    size_t step_staged = 0;
    bool shared_table = true;
    // workspace
    DevBuf part_acc, part_ml, final_ml, logits, group_scores, p_split, pf_part_acc, pf_part_ml;
    // optional per-kernel timing
    bool profiling = false, timed = false;
    hipEvent_t ev0 = nullptr, ev1 = nullptr;
    // A mixed step over a 16-bit cache: the single-token sequences' decode kernel runs on a second stream next to the
    // matrix kernel of the chunks (forked and joined with events, so the caller only ever sees the context's stream).
    hipStream_t side = nullptr;
    hipEvent_t ev_fork = nullptr, ev_join = nullptr;
    bool split16 = false;
    // ALiBi (the op's alibi_slopes input): a slope per query head on the device; the tuned kernels have no such term,
    // so a context with slopes runs on the shape-generic kernels
    DevBuf alibi;
    bool has_alibi = false;  // this step: single-token items are listed behind the chunk items and left to the decode kernel
};

// Every tensor (K and V of every layer) is a reserved range of virtual addresses whose front is backed by physical
// memory; growth maps more memory behind what is there, so a tensor's base address never changes and no block moves.
struct pa_kv_cache {
    pa_config cfg{};
    std::string error;
    uint64_t num_blocks = 0;
    std::vector<void*> key, value;      // base addresses (fixed from creation on)
    size_t granularity = 0;             // size of every physical piece: memory is mapped in equal, equally aligned pieces
    // per tensor (2 * layer + (0 = K, 1 = V)): bytes of one block, of address space, and of address space backed by memory
    std::vector<uint64_t> block_bytes;
    std::vector<size_t> reserved, mapped;
    struct Chunk {
        hipMemGenericAllocationHandle_t handle;
        size_t offset, bytes;
    };
    std::vector<std::vector<Chunk>> chunks;  // per tensor
    DevBuf base_table;                  // the 2 * num_layers base addresses, then the tensors' block sizes, for the copy kernel
    DevBuf pairs;                       // (source, destination) list of one copy launch
    uint64_t all_block_bytes() const {  // one block over every tensor
        uint64_t sum = 0;
        for (uint64_t b : block_bytes) sum += b;
        return sum;
    }
    void*& tensor(size_t t) { return (t & 1) ? value[t >> 1] : key[t >> 1]; }
};

namespace {

template <class Obj, class Fn>
int32_t guarded(Obj* obj, Fn&& fn) {
    try {
        fn();
        return PA_OK;
    } catch (const StatusError& e) {
        if (obj) obj->error = e.what(); else g_last_error = e.what();
        return e.code;
    } catch (const std::bad_alloc&) {
        const char* m = "host allocation failed";
        if (obj) obj->error = m; else g_last_error = m;
        return PA_NOT_ALLOCATED;
    } catch (const std::exception& e) {
        if (obj) obj->error = e.what(); else g_last_error = e.what();
        return PA_UNKNOWN_EXCEPTION;
    } catch (...) {
        if (obj) obj->error = "unknown exception"; else g_last_error = "unknown exception";
        return PA_UNKNOWN_EXCEPTION;
    }
}

struct NoObj { std::string error; };

pa::Shape shape_of(const pa_config& c) { return pa::Shape{c.num_heads, c.num_kv_heads, c.head_size, c.block_size}; }
pa::GenericShape generic_shape_of(const pa_config& c) {
    return pa::GenericShape{c.num_heads, c.num_kv_heads, c.head_size, v_head(c), c.block_size, c.kv_cache_dtype, v_dtype(c)};
}
// The append kernel with a row per 16 lanes is built for K and V alike, head size 64, 96, 128 or 256; everything else takes the
// shape-generic one (a wave per row).
bool tuned_append_shape(const pa_config& c) {
    return kv_alike(c) && (c.head_size == 64 || c.head_size == 96 || c.head_size == 128 || c.head_size == 256);
}

const int32_t* table_for(pa_ctx* ctx, int32_t layer) {
    PA_REQUIRE(layer >= 0 && layer < ctx->cfg.num_layers, PA_OUT_OF_BOUNDS, "layer out of range");
    const size_t idx = ctx->shared_table ? 0 : (size_t)layer;
    PA_REQUIRE(idx < ctx->tables.size() && ctx->table_count[idx] == ctx->total_block_ids && ctx->table_ptr[idx],
               PA_PARAMETER_MISMATCH, "block_indices for this layer were not set for the current step");
    return static_cast<const int32_t*>(ctx->table_ptr[idx]);
}

void check_io(pa_ctx* ctx, int32_t layer, const pa_layer_io* io, bool need_kv, bool need_q) {
    PA_REQUIRE(io, PA_INVALID_C_PARAM, "io is null");
    PA_REQUIRE(ctx->step_ready, PA_PARAMETER_MISMATCH, "pa_step_begin has not been called");
    PA_REQUIRE(io->key_cache && io->value_cache && io->num_blocks > 0, PA_INVALID_C_PARAM, "cache tensors missing");
    // the table was validated against the num_blocks of its own call; the cache handed over now must hold its ids too
    (void)table_for(ctx, layer);
    PA_REQUIRE(io->num_blocks >= ctx->table_bound[ctx->shared_table ? 0 : (size_t)layer], PA_OUT_OF_BOUNDS,
               "the cache tensors hold fewer blocks than the block table of this layer refers to");
    if (need_kv) PA_REQUIRE(io->key && io->value, PA_INVALID_C_PARAM, "key/value missing");
    if (need_q) PA_REQUIRE(io->query && io->out, PA_INVALID_C_PARAM, "query/out missing");
    // the kernels move rows in 16-byte pieces (scores as 4-byte values); a pointer off that grid is refused here
    auto on_grid = [](const void* p, uintptr_t a) { return (reinterpret_cast<uintptr_t>(p) & (a - 1)) == 0; };
    PA_REQUIRE(on_grid(io->key_cache, 16) && on_grid(io->value_cache, 16), PA_INVALID_C_PARAM,
               "cache tensors must start at a multiple of 16 bytes");
    if (need_kv) PA_REQUIRE(on_grid(io->key, 16) && on_grid(io->value, 16), PA_INVALID_C_PARAM,
                            "key/value must start at a multiple of 16 bytes");
    if (need_q) PA_REQUIRE(on_grid(io->query, 16) && on_grid(io->out, 16) && on_grid(io->scores, 4), PA_INVALID_C_PARAM,
                           "query/out must start at a multiple of 16 bytes, scores at a multiple of 4");
}

// Descriptors of the u8 decode kernel's workgroups for one block table (host ids), both plans, into the staging copy
// of the table's buffer.
void fill_decode_descs(const pa_ctx* ctx, const int32_t* ids, uint8_t* stage) {
    const int32_t sw = ctx->sliding_window;
    std::vector<int32_t> soff(ctx->B + 1, 0);
    for (int32_t b = 0; b < ctx->B; ++b) soff[b + 1] = soff[b] + ctx->h_past[b] + (ctx->h_sb[b + 1] - ctx->h_sb[b]);
    for (int w = 0; w < 2; ++w) {
        const int32_t nsplit = ctx->dec_plan[w].nsplit;
        pa::DecodeDesc* out = reinterpret_cast<pa::DecodeDesc*>(stage + ctx->desc_off[w]);
        for (size_t i = 0; i < ctx->h_dec.size(); ++i) {
            const int32_t b = ctx->h_dec[i];
            const int32_t kv_len = ctx->h_past[b] + 1;
            const int32_t first = sw > 0 ? std::max(0, kv_len - sw) : 0;
            const int32_t lo = first / 32, hi = (kv_len + 31) / 32;
            const int32_t per = (hi - lo + nsplit - 1) / nsplit;
            const int32_t* tab = ids + ctx->h_bib[b];
            // cache blocks per 32-token tile, and the sequence's last block (a last tile of one 16-token block repeats it)
            // (blocks of 64 tokens or more: one id per tile, that of the block the tile is a part of)
            const int32_t bs = ctx->cfg.block_size, bpt = bs == 16 ? 2 : 1, last_block = (kv_len - 1) / bs;
            const int32_t sub_shift = bs <= 32 ? 0 : __builtin_ctz((unsigned)(bs / 32));
            for (int32_t s = 0; s < nsplit; ++s) {
                pa::DecodeDesc& d = out[i * nsplit + s];
                std::memset(d.pad, 0, sizeof(d.pad));
                d.b = b;
                d.t = ctx->h_sb[b];
                d.kv_len = kv_len;
                d.first = first;
                d.tb = lo + s * per;
                d.te = std::min(hi, d.tb + per);
                d.table_off = ctx->h_bib[b];
                d.score_off = soff[b];
                d.last_id = tab[last_block];
                for (int32_t j = 0; j < 16; ++j)
                    d.ids[j] = bpt * d.tb + j < bpt * d.te ? tab[std::min((bpt * d.tb + j) >> sub_shift, last_block)] : 0;
            }
        }
    }
}

void do_kv_append(pa_ctx* ctx, int32_t layer, const pa_layer_io* io) {
    check_io(ctx, layer, io, true, false);
    const int32_t* table = table_for(ctx, layer);
    if (tuned_append_shape(ctx->cfg))
        HIP_CHECK(pa::launch_kv_append(ctx->stream, ctx->dev, shape_of(ctx->cfg), ctx->cfg.query_dtype,
                                       ctx->cfg.kv_cache_dtype, io->key, io->value, io->key_cache, io->value_cache, table));
    else
        HIP_CHECK(pa::launch_kv_append_generic(ctx->stream, ctx->dev, generic_shape_of(ctx->cfg), ctx->cfg.query_dtype,
                                               io->key, io->value, io->key_cache, io->value_cache, table));
}

// Block sizes the tuned kernels take.  Their tiles are 32 tokens: two 16-token cache blocks, one 32-token block, or a
// 32-token part of a block of 64, 128 or 256 tokens.
bool tuned_block_size(int32_t bs) { return bs >= 16 && bs <= 256 && (bs & (bs - 1)) == 0; }

// Shapes the tuned u8 decode kernel is built for (it takes the single-token sequences of a step).
// (head size 256 with 16-token blocks would spill registers and is left to the shape-generic kernel)
bool decode_u8_shape(const pa_config& c) {
    return kv_alike(c) && c.kv_cache_dtype == PA_U8 && tuned_block_size(c.block_size) &&
           (c.head_size == 64 || c.head_size == 96 || c.head_size == 128 || (c.head_size == 256 && c.block_size >= 32)) &&
           c.num_heads / c.num_kv_heads <= 16;
}

// Shapes the MFMA kernel is built for: 16-bit caches of the query's type, or u8 caches (dequantised on the way to
// LDS).  It takes every sequence the decode kernel does not.
// (head sizes 96 and 256: its one-row-group variants only -- at 256 one workgroup per CU, two blocks of LDS slots fill
// 103 of its 160 KB; the 16-bit decode kernel, the straight-to-LDS variant and the block-sparse estimate are built for
// 64 and 128)
bool narrow_only(const pa_config& c) { return c.head_size == 96 || c.head_size == 256; }
bool mfma_shape(const pa_config& c) {
    return kv_alike(c) && (c.kv_cache_dtype == PA_U8 || c.kv_cache_dtype == c.query_dtype) && tuned_block_size(c.block_size) &&
           (c.head_size == 64 || c.head_size == 128 || narrow_only(c)) && c.num_heads / c.num_kv_heads <= 256;
}

// Shapes the 16-bit decode kernel is built for (single-token sequences of a call that asks for no scores).
bool decode16_shape(const pa_config& c) {
    return kv_alike(c) && c.kv_cache_dtype != PA_U8 && c.kv_cache_dtype == c.query_dtype && tuned_block_size(c.block_size) &&
           (c.head_size == 64 || c.head_size == 96 || c.head_size == 128 || c.head_size == 256) &&
           c.num_heads / c.num_kv_heads <= 16;
}

// The same questions asked of a context: one with ALiBi slopes has no tuned attention kernel.
bool decode_u8_shape(const pa_ctx* ctx) { return !ctx->has_alibi && decode_u8_shape(ctx->cfg); }
bool mfma_shape(const pa_ctx* ctx) { return !ctx->has_alibi && mfma_shape(ctx->cfg); }
bool decode16_shape(const pa_ctx* ctx) { return !ctx->has_alibi && decode16_shape(ctx->cfg); }
// Whether the planned step runs on the matrix kernel (or, a step of single-token sequences over a 16-bit cache, on the
// 16-bit decode kernel, which is launched in its place).  With more than 16 heads per kv head there is no decode
// kernel, and at head sizes 96 and 256 a step of
// single-token sequences alone is then faster on the shape-generic kernel, whose waves share a kv head's rows among the
// group's heads, than in 16-row tiles that hold one group each (64 x 4096 tokens, 32 heads without grouping: 0.88 ms
// against 1.15); with a multi-token sequence in the step the matrix kernel takes all of it.
bool matrix_step(const pa_ctx* ctx) {
    return mfma_shape(ctx) && ctx->n_items > 0 && !(narrow_only(ctx->cfg) && ctx->T == ctx->B && !decode16_shape(ctx));
}
// Whether the planned step's single-token sequences run on the u8 decode kernel: next to the matrix kernel, which
// takes the other sequences, or -- a shape only the decode kernel is built for (head size 256) -- when there are no others.
bool decode_u8_step(const pa_ctx* ctx) {
    return decode_u8_shape(ctx) && !ctx->h_dec.empty() && (mfma_shape(ctx) || (int32_t)ctx->h_dec.size() == ctx->B);
}

// Split-K plan of the decode kernels: workgroups per (sequence, kv head) and the most blocks one walks.
void plan_decode_u8(const pa_ctx* ctx, bool want_scores, int32_t* nsplit_out, int32_t* max_tiles_out,
                    const std::vector<int32_t>* seqs = nullptr, int32_t* waves_out = nullptr) {
    const pa_config& c = ctx->cfg;
    const int32_t G = c.num_heads / c.num_kv_heads;
    int32_t most = 1;
    int64_t all_tiles = 0;
    for (int32_t b : seqs ? *seqs : ctx->h_dec) {
        const int32_t kv = ctx->h_past[b] + 1;
        const int32_t first = ctx->sliding_window > 0 ? std::max(0, kv - ctx->sliding_window) : 0;
        most = std::max(most, (kv + 31) / 32 - first / 32);
        all_tiles += (kv + 31) / 32 - first / 32;
    }
    const bool u8 = c.kv_cache_dtype == PA_U8;
    const int64_t pairs = (int64_t)(seqs ? seqs->size() : ctx->h_dec.size()) * c.num_kv_heads;
    // `slots` workgroups of `waves` waves run at once (a CU's 160 KB of LDS shared between them, allocated in
    // granules: one granule of margin each)
    auto plan = [&](int32_t waves, int32_t slots, int32_t* cap_out) {
        auto lds_of = [&](int32_t tiles) {
            int32_t off;
            return u8 ? pa::decode_u8_lds_bytes(c.head_size, G, tiles, want_scores, waves, &off, c.block_size)
                      : pa::decode16_lds_bytes(c.head_size, G, tiles, want_scores) + pa::decode16_table_bytes(tiles, c.block_size);
        };
        // the score path keeps a split's probabilities in LDS: that bounds the blocks per workgroup
        const size_t budget = (size_t)(160 * 1024 / (slots / 256));
        auto fits = [&](int32_t tiles) { return (lds_of(tiles) + 1279) / 1280 * 1280 <= budget; };
        int32_t cap = most;
        if (want_scores) {
            cap = std::min<int32_t>(most, (int32_t)(budget / (64 * G)));
            while (cap > 1 && !fits(cap)) --cap;
        }
        *cap_out = cap;
        if (waves == 4) {
            // Four-wave workgroups, two to a CU: the count with the shortest estimated launch.  The estimate (us, per
            // 32-token tile of D = 128; fitted to sweeps over batch sizes and contexts of 1024 - 12288 tokens with the
            // count forced, 4 - 5 % rms): a workgroup alone on its CU takes t1 per tile; once workgroups share CUs (more
            // than half the slots taken) the ones that share take t2 and set the pace; all of them together cannot pull
            // more than the memory system gives in this access pattern (`bw`, less when probabilities are kept);
            // whole rounds of workgroups run one after the other and a last, partial round at the pace of its own
            // occupancy; splits pay for the merge and score launch, which grows with the partial rows.  (Against the
            // rule this replaces -- at least one round of workgroups, at least 16 blocks each, rounds 85 % full --
            // batches of 24 to 56 sequences x 8 kv heads run 10 - 26 % faster, because they are not cut at all; full
            // batches and long contexts come out the same within 2 %.)
            // (head size 256 runs one workgroup per CU; a tile of it is two tiles of head size 128 in bytes, which two
            // workgroups sharing a CU take t2 for)
            const bool sc = want_scores;
            const double dscale = c.head_size / 128.0;
            const double t2 = (u8 ? (sc ? 0.525 : 0.468) : (sc ? 1.104 : 1.064)) * dscale;
            const double t1 = slots == 256 ? t2 / 2 : (u8 ? (sc ? 0.316 : 0.276) : (sc ? 0.495 : 0.478)) * dscale;
            const double tile_bytes = 2.0 * 32 * (u8 ? c.head_size + 8 : 2 * c.head_size), bw = sc ? 5.9e6 : 6.97e6;
            const double post_a = u8 ? (sc ? 2.4 : 1.0) : (sc ? 4.2 : 2.8), post_b = u8 ? (sc ? 0.0079 : 0.0066) : (sc ? 0.0050 : 0.0046);
            auto t_tile = [&](int64_t w) {  // per tile, with w workgroups running at once
                return std::max(w <= slots / 2 || slots == 256 ? t1 : t2, (double)w * tile_bytes / bw);
            };
            // Contexts of unequal length: every sequence is cut into the same number of parts, so its workgroups are
            // as much shorter than the longest one's as its context is; the launch then behaves like one of fewer
            // workgroups of the longest kind (16 sequences x 64 - 2048 positions, D = 64: 6 parts instead of 3, the step
            // 17.2 -> 16.4 us, 12.5 -> 11.2 us without scores; equal contexts are not touched).
            const double fill = (double)all_tiles / ((double)most * (double)(pairs / c.num_kv_heads));
            int32_t best_n = 0;
            double best_t = 0.0;
            for (int32_t n = 1; n <= std::min(most, 64); ++n) {
                const int32_t per = (most + n - 1) / n;
                if (per > cap) continue;
                const int64_t w = pairs * n, w_run = std::max<int64_t>(1, std::llround((double)w * fill));
                const int64_t full = w_run / slots, rem = w_run % slots;
                // (a cut that fills its rounds exactly is preferred over one that does not at equal estimates: the
                // estimate of a partly filled round is the less certain one -- 8 x 32769 runs 2 % faster in 8 than in 7)
                const double t = ((double)full * per * t_tile(slots) + (rem > 0 ? per * t_tile(rem) : 0.0)) *
                                     (n > 1 && rem > 0 ? 1.02 : 1.0) +
                                 (n > 1 ? post_a + post_b * (double)w : 0.0);
                if (best_n == 0 || t < best_t) {
                    best_n = n;
                    best_t = t;
                }
            }
            if (best_n > 0) return best_n;
        }
        // (eight-wave workgroups, one to a CU, and contexts that fit no count up to 64)
        int32_t s = 1;
        // aim for at least one round of workgroups, keep at least 16 blocks per workgroup (with fewer, what the
        // extra workgroups gain is lost again in the merge and score kernels)
        while (pairs * s < slots && most / (s + 1) >= 16) ++s;
        while ((most + s - 1) / s > cap) ++s;
        // more than one round of workgroups: a last round that is mostly empty costs a whole round's time; take
        // more splits until the rounds are at least 85 % full (sequences of one length, the worst case, in mind)
        auto fill = [&](int32_t n) {
            const int64_t w = pairs * n;
            return (double)w / (double)(slots * ((w + slots - 1) / slots));
        };
        if (s > 1 && pairs * s > slots)
            while (fill(s) < 0.85 && most / (s + 1) >= 16) ++s;
        return s;
    };
    int32_t cap4 = 0, waves = 4;
    int32_t s = plan(4, c.head_size > 128 ? 256 : 512, &cap4);
    // A context whose probabilities do not fit half a CU's LDS is cut into splits that send every head's
    // probabilities through HBM and add a merge.  With enough (sequence, kv head) pairs to give every CU a workgroup
    // of its own, one workgroup of eight waves per CU (the same waves per CU, the whole LDS) needs fewer of them.
    if (u8 && c.block_size >= 32 && c.head_size != 96 && c.head_size <= 128 && most > cap4 && pairs >= 256) {
        int32_t cap8 = 0;
        const int32_t s8 = plan(8, 256, &cap8);
        if (s8 < s) {
            s = s8;
            waves = 8;
        }
    }
    *nsplit_out = s;
    *max_tiles_out = (most + s - 1) / s;
    if (waves_out) *waves_out = waves;
}

int xatt_seq_index(const pa_ctx* ctx, int32_t b) { return ctx->h_xseq_of.empty() ? -1 : ctx->h_xseq_of[b]; }

pa::XattDev xatt_dev(const pa_ctx* ctx) {
    pa::XattDev d{};
    if (ctx->h_xseq.empty()) return d;  // seq_of stays null: every sequence is dense
    d.seqs = ctx->x_plan.as<pa::XattSeq>();
    d.seq_of = reinterpret_cast<const int32_t*>(static_cast<const uint8_t*>(ctx->x_plan.p) + ctx->x_seq_of_off);
    d.mask = ctx->x_mask.as<uint32_t>();
    d.item_tiles = ctx->x_item_keep.as<int32_t>();
    d.tiles_stride = ctx->x_keep_words;
    d.xb_shift = __builtin_ctz((unsigned)ctx->xatt_block);
    return d;
}

// Work items of the MFMA kernel: tiles of QT query tokens (QT x G <= 128 rows) against ranges of KV blocks sized so
// that the launch has several hundred workgroups of comparable length.  Listed as: items with more than 16 query
// rows (u8 caches), the other dense ones, then the items of block-sparse sequences.
// A piece of the pinned staging area for an upload of `bytes` that the caller fills and queues on the context's stream.
// With the area used up, the copies queued so far are waited for here and the area starts over (larger: it grows
// until a whole step's pieces fit, up to 32 MiB -- beyond that a step pays such a wait now and then).
uint8_t* stage_piece(pa_ctx* ctx, size_t bytes) {
    const size_t need = (std::max<size_t>(bytes, 1) + 63) & ~(size_t)63;
    if (ctx->step_staged + need > ctx->step_staging.cap) {
        HIP_CHECK(hipStreamSynchronize(ctx->stream));
        ctx->step_staged = 0;
        ctx->step_staging.reserve(std::max<size_t>({need, (size_t)1 << 16, std::min<size_t>(2 * ctx->step_staging.cap, (size_t)32 << 20)}));
    }
    uint8_t* at = ctx->step_staging.as<uint8_t>() + ctx->step_staged;
    ctx->step_staged += need;
    return at;
}

// Queues a copy of `bytes` of host memory to `dst` on the context's stream through the staging area (from a pageable
// source the runtime stages and waits per call, 15 - 20 us per array); `src` is free when this returns.
void stage_upload(pa_ctx* ctx, void* dst, const void* src, size_t bytes) {
    if (bytes == 0) return;
    uint8_t* at = stage_piece(ctx, bytes);
    std::memcpy(at, src, bytes);
    HIP_CHECK(hipMemcpyAsync(dst, at, bytes, hipMemcpyHostToDevice, ctx->stream));
}

void plan_items(pa_ctx* ctx) {
    const int32_t B = ctx->B, T = ctx->T;
    const int32_t* past = ctx->h_past.data();
    const int32_t* sb = ctx->h_sb.data();
    const int32_t G = ctx->cfg.num_heads / ctx->cfg.num_kv_heads;
    // 16-bit caches: every dense item goes to one kernel variant (16 rows per wave, four waves per SIMD; chunk-only
    // launches to the straight-to-LDS variant).  u8 caches: items with more than 16 rows go to a variant of their own
    // (32 rows per wave, two waves per SIMD) and are listed first
    const bool narrow_all = ctx->cfg.kv_cache_dtype != PA_U8;
    const bool no_wide = narrow_all || narrow_only(ctx->cfg);  // (the 32-rows-per-wave u8 variant: head size 64 / 128)
    const int32_t QT = std::max(1, 128 / G), QTX = std::max(1, 128 / G), sw = ctx->sliding_window;
    struct Tile { int32_t b, q0, nq, lo, hi, kind; };  // kind 0: more than 16 rows, 1: the rest, 2: single-token sequences, 3: block-sparse
    std::vector<int32_t> single_idx(B, -1);
    int32_t n_single_seqs = 0;
    std::vector<Tile> tiles;
    int64_t total_blocks = 0;
    const bool split_off_decode = decode_u8_shape(ctx);
    ctx->h_dec.clear();
    ctx->h_dec16.clear();
    // A mixed step over a 16-bit cache with the 16-bit decode kernel available: chunk items and single-token
    // sequences do not share a launch -- the chunks go to the straight-to-LDS variant (head size 128; else the
    // one-row-group variant), the single-token sequences to the decode kernel on a second stream, side by side
    // (60 single tokens at 512 - 8192 positions beside four 512-token chunks over f16, against one launch for both:
    // head size 128 0.296 -> 0.283 ms, 64 0.226 -> 0.213, 96 0.806 -> 0.787; at 256 no difference, left as one launch).  Their items are still listed (behind the chunks' items, where
    // the matrix kernel passes them over) but count for nothing in the plan of the chunks.
    {
        bool any_single = false, any_chunk = false;
        for (int32_t b = 0; b < B; ++b) {
            const int32_t q_len = sb[b + 1] - sb[b];
            any_single = any_single || q_len == 1;
            any_chunk = any_chunk || (q_len > 1 && xatt_seq_index(ctx, b) < 0);
        }
        ctx->split16 = narrow_all && any_single && any_chunk && decode16_shape(ctx) && ctx->cfg.head_size != 256;
    }
    size_t planned_tiles = 0;
    for (int32_t b = 0; b < B; ++b) {
        const int32_t q_len = sb[b + 1] - sb[b];
        if (split_off_decode && q_len == 1) {
            ctx->h_dec.push_back(b);
            continue;
        }
        const bool sparse = xatt_seq_index(ctx, b) >= 0;
        const int32_t qt = sparse ? QTX : QT;
        if (q_len == 1) ctx->h_dec16.push_back(b);
        if (q_len == 1) single_idx[b] = n_single_seqs++;
        for (int32_t q0 = 0; q0 < q_len; q0 += qt) {
            const int32_t nq = std::min(qt, q_len - q0);
            const int32_t last_pos = past[b] + q0 + nq - 1;
            const int32_t first_pos = sw > 0 ? std::max(0, past[b] + q0 + 1 - sw) : 0;
            tiles.push_back({b, q0, nq, first_pos / 32, last_pos / 32 + 1, sparse ? 3 : q_len == 1 ? 2 : (nq * G > 16 ? 0 : 1)});
            if (q_len == 1 && ctx->split16) continue;  // (another kernel's work)
            total_blocks += last_pos / 32 + 1 - first_pos / 32;
            ++planned_tiles;
        }
    }
    // Ranges of at least 8 blocks -- of at least 16 once the uncut tiles alone make three quarters of a round of
    // workgroups: cutting their short items further adds workgroups nobody waits for and a merge pass for their rows
    // (four 512-token prompts from scratch: 42.8 -> 33.6 us over bf16, 56.5 -> 44.4 us over u8; a single one, whose 116
    // to 128 workgroups leave most of the chip idle, is better off cut: 29.9 against 35.2 us over u8).
    const bool round_filled = (int64_t)planned_tiles * ctx->cfg.num_kv_heads >= 384;
    const int64_t shortest = round_filled ? 16 : 8;
    int64_t target = std::min<int64_t>(128, std::max<int64_t>(shortest, total_blocks * ctx->cfg.num_kv_heads / 768));
    // ... and tiles of about one length that fill the round by themselves are not cut at all: there is nothing to
    // balance (32 sequences x 64 tokens behind 500: 62.6 -> 42.6 us over bf16, 77.2 -> 56.1 us over u8)
    if (round_filled && !tiles.empty()) {
        int64_t longest = 0;
        for (const Tile& t : tiles)
            if (!(t.kind == 2 && ctx->split16)) longest = std::max<int64_t>(longest, t.hi - t.lo);
        if (2 * longest * (int64_t)planned_tiles <= 3 * total_blocks) target = std::min<int64_t>(128, std::max(target, longest));
    }
    // single-token sequences as items of the kernel variant that can hand their probabilities to the score kernel
    const bool stash_ok = narrow_all && G <= 16;
    ctx->stash_ok = stash_ok;
    std::vector<pa::PrefillItem>& items = ctx->h_items;
    items.clear();
    std::vector<int32_t> tok_ns(T, 1);
    int32_t max_split = 1, longest_sparse = 1;
    std::stable_sort(tiles.begin(), tiles.end(), [](const Tile& x, const Tile& y) { return x.kind < y.kind; });
    ctx->n_wide = 0;
    ctx->n_sparse = 0;
    ctx->n_single = 0;
    for (const Tile& t : tiles) {
        const int32_t nt = t.hi - t.lo;
        // (items of single-token sequences over 16-bit caches keep their probabilities in LDS when scores are wanted)
        const int64_t most = t.kind == 2 && stash_ok ? std::min<int64_t>(target, pa::single_item_max_tiles(G)) : target;
        const int32_t per = (int32_t)((nt + (nt + most - 1) / most - 1) / ((nt + most - 1) / most));
        const int32_t ns = (nt + per - 1) / per;
        for (int32_t s = 0; s < ns; ++s)
            items.push_back({t.b, t.q0, t.nq, t.lo + s * per, std::min(t.hi, t.lo + (s + 1) * per), s, ns, 0});
        if (t.kind == 0 && !no_wide) ctx->n_wide += ns;
        if (t.kind == 2) ctx->n_single += ns;
        if (t.kind == 3) {
            ctx->n_sparse += ns;
            longest_sparse = std::max(longest_sparse, per);
        }
        for (int32_t i = 0; i < t.nq; ++i) tok_ns[sb[t.b] + t.q0 + i] = ns;
        max_split = std::max(max_split, ns);
    }
    // Workgroups start in list order and a CU slot works through two or three of them in a launch: the dense items of
    // multi-token sequences are listed longest first (within the wide and the narrow group), so that no long item
    // starts last and finishes alone.
    {
        auto longer = [](const pa::PrefillItem& x, const pa::PrefillItem& y) { return x.te - x.tb > y.te - y.tb; };
        const int32_t n_multi = (int32_t)items.size() - ctx->n_sparse - ctx->n_single;
        std::stable_sort(items.begin(), items.begin() + ctx->n_wide, longer);
        std::stable_sort(items.begin() + ctx->n_wide, items.begin() + n_multi, longer);
    }
    PA_REQUIRE(longest_sparse <= 128, PA_UNKNOWN_EXCEPTION, "a block-sparse work item walks more than 128 KV blocks");
    // A mixed step over a 16-bit cache runs the single-token items (bandwidth-bound) and the chunk items
    // (matrix-bound) in one launch of one kernel variant.  Workgroups start in list order, so the two kinds only share
    // the CUs if the list alternates between them.  A few single-token items are best left at the end, where they
    // fill the tail behind the last long chunk items; once they add up to more than about a third of the chunk
    // items' time (measured: 11 ns per KV block of a single-token item, 1.9 ns per KV block and 16 query rows of a
    // chunk item, per kv head), the chunk items are spread over the first half of the list with every second
    // single-token item between them.  Spreading them over the whole list lets a chunk item start last and finish
    // alone; over less than half leaves a long bandwidth-bound tail.  (Config 3: 0.274 -> 0.251 ms; with 28 or fewer
    // single-token sequences next to the same chunks the plain order is 1 % faster.)
    {
        const int32_t n_multi = (int32_t)items.size() - ctx->n_sparse - ctx->n_single, n_s = ctx->n_single;
        double cost_m = 0, cost_s = 0;
        for (int32_t i = 0; i < n_multi; ++i) cost_m += 1.9 * (items[i].te - items[i].tb) * ((items[i].nq * G + 15) / 16);
        for (int32_t i = 0; i < n_s; ++i) cost_s += 11.0 * (items[n_multi + i].te - items[n_multi + i].tb);
        // (the single-token items longest first as well: 0.272 -> 0.266 ms on the same workload)
        std::stable_sort(items.begin() + n_multi, items.begin() + n_multi + n_s,
                         [](const pa::PrefillItem& x, const pa::PrefillItem& y) { return x.te - x.tb > y.te - y.tb; });
        if (narrow_all && n_s > 0 && n_multi > 0 && cost_s > 0.3 * cost_m && !ctx->split16) {
            std::vector<pa::PrefillItem> mixed;
            mixed.reserve(items.size());
            int32_t im = 0, is = 0;
            while (im < n_multi || is < n_s) {
                const bool take_multi = im < n_multi && (is >= n_s || (int64_t)im * n_s <= 2 * (int64_t)is * n_multi);
                mixed.push_back(take_multi ? items[im++] : items[n_multi + is++]);
            }
            mixed.insert(mixed.end(), items.begin() + n_multi + n_s, items.end());
            items.swap(mixed);
        }
    }
    // The decode kernels' workgroups start in list order too: longest contexts first (equal lengths keep their order, and
    // a list that is 0, 1, 2, ... is not passed at all)
    {
        auto longer = [&](int32_t x, int32_t y) { return past[x] > past[y]; };
        std::stable_sort(ctx->h_dec.begin(), ctx->h_dec.end(), longer);
        std::stable_sort(ctx->h_dec16.begin(), ctx->h_dec16.end(), longer);
        auto identity = [&](const std::vector<int32_t>& v) {
            if ((int32_t)v.size() != B) return false;
            for (int32_t i = 0; i < B; ++i)
                if (v[i] != i) return false;
            return true;
        };
        ctx->dec_in_order = identity(ctx->h_dec);
        ctx->dec16_in_order = identity(ctx->h_dec16);
    }
    ctx->x_keep_words = 1 + longest_sparse;  // entries of a work item's block list
    ctx->n_items = (int32_t)items.size();
    ctx->max_split = max_split;
    const size_t item_bytes = items.size() * sizeof(pa::PrefillItem);
    // one upload: items | split count per token | single-token index per sequence (-1 for the others) | the tokens
    // whose rows the merge kernel has to fold
    ctx->n_merge = 0;
    for (int32_t t = 0; t < T; ++t) ctx->n_merge += tok_ns[t] > 1;
    tok_ns.insert(tok_ns.end(), single_idx.begin(), single_idx.end());
    for (int32_t t = 0; t < T; ++t)
        if (tok_ns[t] > 1) tok_ns.push_back(t);
    ctx->single_idx_off = item_bytes + (size_t)T * sizeof(int32_t);
    ctx->merge_tok_off = ctx->single_idx_off + (size_t)B * sizeof(int32_t);
    ctx->items.reserve(item_bytes + tok_ns.size() * sizeof(int32_t));
    stage_upload(ctx, ctx->items.p, items.data(), item_bytes);
    stage_upload(ctx, static_cast<uint8_t*>(ctx->items.p) + item_bytes, tok_ns.data(), tok_ns.size() * sizeof(int32_t));
    // the sequences a score replay has rows for: those with more than one token, longest context first
    ctx->h_multi.clear();
    for (int32_t b = 0; b < B; ++b)
        if (sb[b + 1] - sb[b] > 1) ctx->h_multi.push_back(b);
    std::stable_sort(ctx->h_multi.begin(), ctx->h_multi.end(),
                     [&](int32_t x, int32_t y) { return past[x] + sb[x + 1] - sb[x] > past[y] + sb[y + 1] - sb[y]; });
    if (!ctx->h_multi.empty()) {
        ctx->multi_list.reserve(ctx->h_multi.size() * sizeof(int32_t));
        stage_upload(ctx, ctx->multi_list.p, ctx->h_multi.data(), ctx->h_multi.size() * sizeof(int32_t));
    }
    if (!ctx->h_dec16.empty()) {
        ctx->dec16_list.reserve(ctx->h_dec16.size() * sizeof(int32_t));
        stage_upload(ctx, ctx->dec16_list.p, ctx->h_dec16.data(), ctx->h_dec16.size() * sizeof(int32_t));
    }
    if (!ctx->h_dec.empty()) {
        ctx->dec_list.reserve(ctx->h_dec.size() * sizeof(int32_t));
        stage_upload(ctx, ctx->dec_list.p, ctx->h_dec.data(), ctx->h_dec.size() * sizeof(int32_t));
    }
    ctx->tok_nsplit_off = item_bytes;
    if (split_off_decode && !ctx->h_dec.empty())
        for (int w = 0; w < 2; ++w)
            plan_decode_u8(ctx, w == 1, &ctx->dec_plan[w].nsplit, &ctx->dec_plan[w].max_tiles, nullptr, &ctx->dec_plan[w].waves);
}

// Workspace of a decode launch (split partials, final maxima and denominators, per-kv-head score sums or per-head
// split probabilities): the context's growable buffers, or -- from_static -- pieces of the fixed device scratch, in
// which case nothing is allocated and a step that needs more than the scratch holds is refused.
struct DecodeWs {
    float *part_acc, *part_ml, *final_ml;
    _Float16 *group_scores, *p_split;
};

DecodeWs decode_workspace(pa_ctx* ctx, size_t rows, int32_t nsplit, bool want_scores, bool from_static) {
    const pa_config& c = ctx->cfg;
    const size_t b_final = rows * 2 * sizeof(float);
    const size_t b_acc = nsplit > 1 ? rows * nsplit * c.head_size * sizeof(float) : 0;
    const size_t b_ml = nsplit > 1 ? rows * nsplit * 2 * sizeof(float) : 0;
    const size_t b_group = want_scores && nsplit == 1 ? (size_t)c.num_kv_heads * ctx->total_scores * sizeof(uint16_t) : 0;
    const size_t b_psplit = want_scores && nsplit > 1
                                ? (size_t)c.num_heads * pa::p_split_stride(ctx->total_scores, ctx->B) * sizeof(uint16_t) : 0;
    DecodeWs w{};
    if (from_static) {
        size_t off = 0;
        auto place = [&](size_t bytes) {
            const size_t at = off;
            off += (bytes + 255) & ~(size_t)255;
            return at;
        };
        const size_t o_final = place(b_final), o_acc = place(b_acc), o_ml = place(b_ml), o_group = place(b_group),
                     o_psplit = place(b_psplit);
        PA_REQUIRE(off <= STATIC_SCRATCH_BYTES, PA_OUT_OF_BOUNDS,
                   "pa_attention_static: this step needs " + std::to_string(off) + " bytes of workspace, the fixed scratch holds " +
                       std::to_string(STATIC_SCRATCH_BYTES) + " (use pa_attention)");
        PA_REQUIRE(ctx->static_scratch, PA_NOT_ALLOCATED, "the fixed scratch of this device was not resolved");
        uint8_t* base = ctx->static_scratch;
        w.final_ml = reinterpret_cast<float*>(base + o_final);
        w.part_acc = reinterpret_cast<float*>(base + o_acc);
        w.part_ml = reinterpret_cast<float*>(base + o_ml);
        w.group_scores = reinterpret_cast<_Float16*>(base + o_group);
        w.p_split = reinterpret_cast<_Float16*>(base + o_psplit);
        return w;
    }
    ctx->final_ml.reserve(b_final);
    if (b_acc) ctx->part_acc.reserve(b_acc);
    if (b_ml) ctx->part_ml.reserve(b_ml);
    if (b_group) ctx->group_scores.reserve(b_group);
    if (b_psplit) ctx->p_split.reserve(b_psplit);
    w.final_ml = ctx->final_ml.as<float>();
    w.part_acc = ctx->part_acc.as<float>();
    w.part_ml = ctx->part_ml.as<float>();
    w.group_scores = ctx->group_scores.as<_Float16>();
    w.p_split = ctx->p_split.as<_Float16>();
    return w;
}

// fuse_append: the call is the attention half of pa_forward in a step whose sequences all go to one decode kernel (the
// u8 one or the 16-bit one), and no append kernel has run: the decode kernel writes the step's K / V rows itself.
void do_attention(pa_ctx* ctx, int32_t layer, const pa_layer_io* io, bool static_ws = false, bool fuse_append = false) {
    check_io(ctx, layer, io, false, true);
    const int32_t* table = table_for(ctx, layer);
    const pa_config& c = ctx->cfg;
    const size_t rows = (size_t)ctx->T * c.num_heads;
    const bool use_decode = decode_u8_step(ctx);
    const bool use_mfma = matrix_step(ctx);
    // 16-bit caches, no dense chunk in the step: the single-token sequences go to their own decode kernel.  (Next to
    // dense chunks they stay work items of the matrix kernel: bandwidth-bound and matrix-bound items share the CUs
    // inside one launch, which two launches one after the other do not.)
    const bool side_by_side = ctx->split16 && !static_ws;
    const bool use_decode16 = use_mfma && decode16_shape(ctx) && !ctx->h_dec16.empty() &&
                              (ctx->n_single + ctx->n_sparse == ctx->n_items || side_by_side);
    const bool mfma_left = use_mfma && !(use_decode16 && ctx->n_single == ctx->n_items);
    if (static_ws)
        PA_REQUIRE((use_decode && (int32_t)ctx->h_dec.size() == ctx->B) || (use_decode16 && !mfma_left && !use_decode),
                   PA_NOT_IMPLEMENTED,
                   "pa_attention_static serves steps in which every sequence schedules one token, over a u8 cache or a "
                   "16-bit cache of the query's type (block size 16 to 256, a power of two; head size 64, 96, 128 or 256 -- over u8 with 16-token blocks not 256 --, K and V alike; at most 16 heads per kv head)");
    // the timed kernel: the matrix kernel when there is prefill work, else the decode kernel
    hipEvent_t ev0 = ctx->profiling ? ctx->ev0 : nullptr, ev1 = ctx->profiling ? ctx->ev1 : nullptr;
    // fork: what is launched on the returned stream starts behind what the context's stream holds so far and runs
    // next to what follows on it, until the join at the end of this call
    bool forked = false;
    auto fork_side = [&]() -> hipStream_t {
        if (!ctx->side) {
            HIP_CHECK(hipStreamCreateWithFlags(&ctx->side, hipStreamNonBlocking));
            HIP_CHECK(hipEventCreateWithFlags(&ctx->ev_fork, hipEventDisableTiming));
            HIP_CHECK(hipEventCreateWithFlags(&ctx->ev_join, hipEventDisableTiming));
        }
        if (!forked) {
            HIP_CHECK(hipEventRecord(ctx->ev_fork, ctx->stream));
            HIP_CHECK(hipStreamWaitEvent(ctx->side, ctx->ev_fork, 0));
            forked = true;
        }
        return ctx->side;
    };
    if (use_decode) {
        pa::DecodeArgs a{};
        a.st = ctx->dev;
        a.sh = shape_of(c);
        a.G = c.num_heads / c.num_kv_heads;
        a.want_scores = io->scores ? 1 : 0;
        a.total_scores = ctx->total_scores;
        const int wplan = io->scores ? 1 : 0;
        a.nsplit = ctx->dec_plan[wplan].nsplit;
        a.max_tiles = ctx->dec_plan[wplan].max_tiles;
        a.waves = ctx->dec_plan[wplan].waves;
        a.descs = reinterpret_cast<const pa::DecodeDesc*>(reinterpret_cast<const uint8_t*>(table) + ctx->desc_off[wplan]);
        a.key = static_cast<const uint16_t*>(io->key);
        a.value = static_cast<const uint16_t*>(io->value);
        a.fuse_append = fuse_append ? 1 : 0;
        a.n_seqs = (int32_t)ctx->h_dec.size();
        a.seq_list = ctx->dec_in_order ? nullptr : ctx->dec_list.as<int32_t>();
        ctx->nsplit = a.nsplit;
        const DecodeWs ws = decode_workspace(ctx, rows, a.nsplit, io->scores != nullptr, static_ws);
        a.query = static_cast<const uint16_t*>(io->query);
        a.key_cache = static_cast<const uint8_t*>(io->key_cache);
        a.value_cache = static_cast<const uint8_t*>(io->value_cache);
        a.block_indices = table;
        a.out = static_cast<uint16_t*>(io->out);
        a.part_acc = ws.part_acc;
        a.part_ml = ws.part_ml;
        a.final_ml = ws.final_ml;
        a.group_scores = ws.group_scores;
        a.p_split = ws.p_split;
        // (next to the matrix kernel of a mixed step: on the second stream, like the 16-bit decode kernel below)
        HIP_CHECK(pa::launch_decode_u8(use_mfma && !static_ws ? fork_side() : ctx->stream, a, c.query_dtype, io->scores,
                                       ctx->max_kv, use_mfma ? nullptr : ev0, use_mfma ? nullptr : ev1));
        ctx->timed = ctx->profiling;
    }
    if (use_decode16) {
        pa::DecodeArgs a{};
        a.st = ctx->dev;
        a.sh = shape_of(c);
        a.G = c.num_heads / c.num_kv_heads;
        a.want_scores = io->scores ? 1 : 0;
        a.total_scores = ctx->total_scores;
        plan_decode_u8(ctx, io->scores != nullptr, &a.nsplit, &a.max_tiles, &ctx->h_dec16);
        a.waves = 4;
        a.key = static_cast<const uint16_t*>(io->key);
        a.value = static_cast<const uint16_t*>(io->value);
        a.fuse_append = fuse_append ? 1 : 0;
        a.n_seqs = (int32_t)ctx->h_dec16.size();
        a.seq_list = ctx->dec16_in_order ? nullptr : ctx->dec16_list.as<int32_t>();
        ctx->nsplit = a.nsplit;
        const DecodeWs ws = decode_workspace(ctx, rows, a.nsplit, io->scores != nullptr, static_ws);
        a.query = static_cast<const uint16_t*>(io->query);
        a.key_cache = static_cast<const uint8_t*>(io->key_cache);
        a.value_cache = static_cast<const uint8_t*>(io->value_cache);
        a.block_indices = table;
        a.out = static_cast<uint16_t*>(io->out);
        a.part_acc = ws.part_acc;
        a.part_ml = ws.part_ml;
        a.final_ml = ws.final_ml;
        a.group_scores = ws.group_scores;
        a.p_split = ws.p_split;
        HIP_CHECK(pa::launch_decode16(side_by_side ? fork_side() : ctx->stream, a, c.query_dtype, io->scores, ctx->max_kv,
                                      mfma_left ? nullptr : ev0, mfma_left ? nullptr : ev1));
        ctx->timed = ctx->profiling;
    }
    if (mfma_left) {
        pa::PrefillArgs a{};
        a.skip_single = use_decode16 ? 1 : 0;
        a.st = ctx->dev;
        a.sh = shape_of(c);
        a.query = static_cast<const uint16_t*>(io->query);
        a.key_cache = static_cast<const uint8_t*>(io->key_cache);
        a.value_cache = static_cast<const uint8_t*>(io->value_cache);
        a.block_indices = table;
        a.items = ctx->items.as<pa::PrefillItem>();
        a.tok_nsplit = reinterpret_cast<const int32_t*>(static_cast<const uint8_t*>(ctx->items.p) + ctx->tok_nsplit_off);
        a.n_items = ctx->n_items;
        a.n_wide = ctx->n_wide;
        a.G = c.num_heads / c.num_kv_heads;
        a.max_split = ctx->max_split;
        a.out = static_cast<uint16_t*>(io->out);
        ctx->final_ml.reserve(rows * 2 * sizeof(float));
        a.final_ml = ctx->final_ml.as<float>();
        if (ctx->max_split > 1) {
            ctx->pf_part_acc.reserve(rows * ctx->max_split * c.head_size * sizeof(float));
            ctx->pf_part_ml.reserve(rows * ctx->max_split * 2 * sizeof(float));
        }
        a.part_acc = ctx->pf_part_acc.as<float>();
        a.part_ml = ctx->pf_part_ml.as<float>();
        a.n_sparse = ctx->n_sparse;
        a.xatt = xatt_dev(ctx);
        a.n_single = ctx->n_single;
        a.single_idx = reinterpret_cast<const int32_t*>(static_cast<const uint8_t*>(ctx->items.p) + ctx->single_idx_off);
        a.merge_tokens = reinterpret_cast<const int32_t*>(static_cast<const uint8_t*>(ctx->items.p) + ctx->merge_tok_off);
        a.n_merge = ctx->n_merge;
        if (ctx->n_sparse > 0) {  // importance estimate and block selection of the block-sparse sequences
            pa::XattArgs x{};
            x.st = ctx->dev;
            x.sh = a.sh;
            x.query = a.query;
            x.key_cache = a.key_cache;
            x.block_indices = table;
            x.seqs = a.xatt.seqs;
            x.seq_of = a.xatt.seq_of;
            x.tiles = reinterpret_cast<const pa::XattTile*>(static_cast<const uint8_t*>(ctx->x_plan.p) + ctx->x_tiles_off);
            x.nseq = (int32_t)ctx->h_xseq.size();
            x.ntiles = ctx->x_ntiles;
            x.max_nqs = ctx->x_max_nqs;
            x.max_nqb = ctx->x_max_nqb;
            x.max_nkb = ctx->x_max_nkb;
            x.xb_shift = a.xatt.xb_shift;
            x.s_shift = __builtin_ctz((unsigned)ctx->xatt_stride);
            x.logits = ctx->x_logits.as<float>();
            x.sums = ctx->x_sums.as<float>();
            x.mask = ctx->x_mask.as<uint32_t>();
            x.items = a.items + (ctx->n_items - ctx->n_sparse);
            x.n_items = ctx->n_sparse;
            x.item_tiles = ctx->x_item_keep.as<int32_t>();
            x.tiles_stride = ctx->x_keep_words;
            x.G = a.G;
            HIP_CHECK(pa::launch_xattention(ctx->stream, x, c.query_dtype, c.kv_cache_dtype));
            ctx->x_ran = true;
        }
        // Single-token sequences that are work items of this launch (16-bit caches, next to dense chunks): with scores
        // wanted the kernel leaves their probabilities for a small score kernel, instead of a replay that reads all
        // their K rows once more.
        const bool hand_over = io->scores && ctx->stash_ok && !use_decode16 && ctx->n_single > 0;
        if (hand_over) {
            const size_t tiles = (size_t)pa::tile_max_count(ctx->total_scores, ctx->B);
            ctx->p_split.reserve(tiles * c.num_heads * 32 * sizeof(uint16_t));
            ctx->tile_max.reserve(tiles * c.num_heads * sizeof(float));
            a.p_out = ctx->p_split.as<_Float16>();
            a.tile_max = ctx->tile_max.as<float>();
        }
        if (!use_decode && !use_decode16) ctx->nsplit = ctx->max_split;
        // scores of the multi-token sequences (and of single-token ones that were work items of this kernel and kept
        // nothing for the score rows): replay; the kept probabilities become scores in extra rows of the same launch,
        // and so does the fold of the rows that were cut into ranges (the score rows fold those rows' maxima and
        // denominators themselves, so nothing in the launch waits for anything else in it)
        const bool score_launch = io->scores && !(use_decode16 && ctx->n_single == ctx->n_items);
        pa::SingleScores ss{};
        if (score_launch && hand_over) {
            ss.p_out = a.p_out;
            ss.tile_max = a.tile_max;
            ss.seq_list = ctx->dec16_list.as<int32_t>();
            ss.n_seqs = (int32_t)ctx->h_dec16.size();
        }
        // (without the single-token sequences the launch has rows for the listed multi-token sequences only)
        const bool singles_too = !(decode_u8_shape(ctx) || use_decode16 || hand_over);
        const int32_t replay_seqs = singles_too ? ctx->B : (int32_t)ctx->h_multi.size();
        const bool merge_later = score_launch && a.n_merge > 0 && replay_seqs + ss.n_seqs > 0 && ctx->max_kv > 0;
        HIP_CHECK(pa::launch_prefill16(ctx->stream, a, c.query_dtype, c.kv_cache_dtype, ev0, ev1, merge_later));
        ctx->timed = ctx->profiling;
        if (score_launch) {
            pa::MergeRows mg{};
            if (merge_later) mg = pa::merge_rows_of(a);
            HIP_CHECK(pa::launch_scores_replay(ctx->stream, ctx->dev, a.sh, c.query_dtype, c.kv_cache_dtype, io->query,
                                               io->key_cache, table, a.final_ml, io->scores, ctx->max_kv,
                                               singles_too ? nullptr : ctx->multi_list.as<int32_t>(), replay_seqs,
                                               a.xatt, ss, mg));
        }
    }
    if (forked) {  // join
        HIP_CHECK(hipEventRecord(ctx->ev_join, ctx->side));
        HIP_CHECK(hipStreamWaitEvent(ctx->stream, ctx->ev_join, 0));
    }
    if (use_decode || use_mfma) return;  // (use_decode16 implies use_mfma)
    ctx->nsplit = ctx->generic_nsplit;
    ctx->part_acc.reserve(rows * ctx->nsplit * v_head(c) * sizeof(float));
    ctx->part_ml.reserve(rows * ctx->nsplit * 2 * sizeof(float));
    ctx->final_ml.reserve(rows * 2 * sizeof(float));
    if (io->scores) ctx->logits.reserve((size_t)c.num_heads * ctx->total_scores * sizeof(float));
    pa::AttnWorkspace ws{ctx->part_acc.as<float>(), ctx->part_ml.as<float>(), ctx->final_ml.as<float>(),
                         ctx->logits.as<float>(), ctx->nsplit, ctx->total_scores,
                         ctx->has_alibi ? ctx->alibi.as<float>() : nullptr};
    HIP_CHECK(pa::launch_attention_generic(ctx->stream, ctx->dev, generic_shape_of(c), c.query_dtype,
                                           io->query, io->key_cache, io->value_cache, table, ws, io->out, io->scores,
                                           ctx->max_kv, ctx->profiling ? ctx->ev0 : nullptr,
                                           ctx->profiling ? ctx->ev1 : nullptr));
    ctx->timed = ctx->profiling;
}

}  // namespace

extern "C" {

const char* pa_version(void) { return "pa_amd 0.1 (gfx950)"; }
const char* pa_global_last_error(void) { return g_last_error.c_str(); }

int32_t pa_create(const pa_config* cfg, pa_ctx** out) {
    return guarded<NoObj>(nullptr, [&] {
        PA_REQUIRE(out, PA_INVALID_C_PARAM, "out is null");
        *out = nullptr;
        check_config(cfg);
        HIP_CHECK(hipSetDevice(cfg->device));
        uint8_t* fixed = static_cast<uint8_t*>(resolve_static_scratch(cfg->device));
        // the decode kernels' device code is uploaded now rather than inside the first attention call (which, for
        // pa_attention_static, must not allocate)
        HIP_CHECK(pa::preload_decode_u8());
        HIP_CHECK(pa::preload_decode16());
        pa_ctx* ctx = new pa_ctx();
        ctx->cfg = *cfg;
        ctx->stream = static_cast<hipStream_t>(cfg->stream);
        ctx->static_scratch = fixed;
        *out = ctx;
    });
}

void pa_destroy(pa_ctx* ctx) {
    if (!ctx) return;
    (void)hipSetDevice(ctx->cfg.device);
    (void)hipStreamSynchronize(ctx->stream);
    ctx->meta.release();
    ctx->items.release();
    for (auto& t : ctx->tables) t.release();
    ctx->table_pool.release();
    ctx->alibi.release();
    ctx->step_staging.release();
    ctx->part_acc.release();
    ctx->part_ml.release();
    ctx->final_ml.release();
    ctx->logits.release();
    ctx->group_scores.release();
    ctx->p_split.release();
    ctx->pf_part_acc.release();
    ctx->pf_part_ml.release();
    ctx->dec_list.release();
    ctx->dec16_list.release();
    ctx->multi_list.release();
    ctx->tile_max.release();
    ctx->trig_lut.release();
    ctx->rot_args.release();
    ctx->div_seqs.release();
    ctx->div_stats.release();
    ctx->div_mean.release();
    ctx->div_colsum.release();
    ctx->x_plan.release();
    ctx->x_logits.release();
    ctx->x_sums.release();
    ctx->x_mask.release();
    ctx->x_item_keep.release();
    if (ctx->side) (void)hipStreamDestroy(ctx->side);
    if (ctx->ev_fork) (void)hipEventDestroy(ctx->ev_fork);
    if (ctx->ev_join) (void)hipEventDestroy(ctx->ev_join);
    if (ctx->ev0) (void)hipEventDestroy(ctx->ev0);
    if (ctx->ev1) (void)hipEventDestroy(ctx->ev1);
    delete ctx;
}

const char* pa_last_error(const pa_ctx* ctx) { return ctx ? ctx->error.c_str() : g_last_error.c_str(); }

int32_t pa_step_begin(pa_ctx* ctx, const pa_step_meta* m) {
    if (!ctx) return PA_INVALID_C_PARAM;
    return guarded(ctx, [&] {
        ctx->step_ready = false;
        PA_REQUIRE(m, PA_INVALID_C_PARAM, "meta is null");
        PA_REQUIRE(m->num_sequences > 0, PA_PARAMETER_MISMATCH, "num_sequences must be positive");
        PA_REQUIRE(m->past_lens && m->subsequence_begins && m->block_indices_begins, PA_INVALID_C_PARAM,
                   "past_lens / subsequence_begins / block_indices_begins missing");
        PA_REQUIRE(m->sliding_window >= 0, PA_PARAMETER_MISMATCH, "sliding_window must be >= 0");
        const int32_t B = m->num_sequences;
        const int32_t bs = ctx->cfg.block_size;
        PA_REQUIRE(m->subsequence_begins[0] == 0 && m->block_indices_begins[0] == 0, PA_PARAMETER_MISMATCH,
                   "subsequence_begins and block_indices_begins must start at 0");
        int64_t total_scores = 0;
        int32_t max_kv = 0;
        for (int32_t b = 0; b < B; ++b) {
            const int64_t q_len = (int64_t)m->subsequence_begins[b + 1] - m->subsequence_begins[b];
            const int64_t nblk = (int64_t)m->block_indices_begins[b + 1] - m->block_indices_begins[b];
            PA_REQUIRE(q_len > 0, PA_PARAMETER_MISMATCH, "every sequence must schedule at least one token");
            PA_REQUIRE(m->past_lens[b] >= 0, PA_PARAMETER_MISMATCH, "past_lens must be >= 0");
            const int64_t kv = (int64_t)m->past_lens[b] + q_len;
            PA_REQUIRE(kv <= INT32_MAX, PA_OUT_OF_BOUNDS, "context length overflows int32");
            PA_REQUIRE(nblk >= (kv + bs - 1) / bs, PA_OUT_OF_BOUNDS,
                       "block table of a sequence is shorter than its context");
            total_scores += kv;
            max_kv = std::max<int32_t>(max_kv, (int32_t)kv);
        }
        PA_REQUIRE(total_scores <= INT32_MAX, PA_OUT_OF_BOUNDS, "sum of context lengths overflows int32");
        const int32_t T = m->subsequence_begins[B];
        const int32_t n_ids = m->block_indices_begins[B];
        PA_REQUIRE((int64_t)T * ctx->cfg.num_heads <= INT32_MAX, PA_OUT_OF_BOUNDS,
                   "tokens x query heads of a step overflow int32");

        // pack the device copy: past | sb | bib | window | score_off | token_seq | token tiles of the generic kernel
        const pa::GenericShape gsh = generic_shape_of(ctx->cfg);
        const pa::GenericPlan gplan = pa::generic_plan(gsh, T > B);
        std::vector<int32_t> h((size_t)B + (B + 1) + (B + 1) + B + (B + 1) + T + T);
        int32_t* past = h.data();
        int32_t* sb = past + B;
        int32_t* bib = sb + B + 1;
        int32_t* win = bib + B + 1;
        int32_t* soff = win + B;
        int32_t* tseq = soff + B + 1;
        std::memcpy(past, m->past_lens, sizeof(int32_t) * B);
        std::memcpy(sb, m->subsequence_begins, sizeof(int32_t) * (B + 1));
        std::memcpy(bib, m->block_indices_begins, sizeof(int32_t) * (B + 1));
        soff[0] = 0;
        for (int32_t b = 0; b < B; ++b) {
            const int32_t q_len = sb[b + 1] - sb[b];
            int32_t w = m->score_aggregation_window ? m->score_aggregation_window[b] : 1;
            PA_REQUIRE(w >= 0, PA_PARAMETER_MISMATCH, "score_aggregation_window must be >= 0");
            win[b] = std::min(w, q_len);
            soff[b + 1] = soff[b] + past[b] + q_len;
            for (int32_t t = sb[b]; t < sb[b + 1]; ++t) tseq[t] = b;
        }
        PA_REQUIRE((int64_t)T * 8 <= INT32_MAX, PA_OUT_OF_BOUNDS, "too many tokens in a step");
        int32_t* gtiles = tseq + T;
        int32_t n_gtiles = 0;
        for (int32_t b = 0; b < B; ++b)
            for (int32_t t = sb[b]; t < sb[b + 1]; t += gplan.tokens)
                gtiles[n_gtiles++] = t * 8 + (std::min(gplan.tokens, sb[b + 1] - t) - 1);

        HIP_CHECK(hipSetDevice(ctx->cfg.device));
        // the previous step's kernels may still read the old copy
        HIP_CHECK(hipStreamSynchronize(ctx->stream));
        ctx->meta.reserve(h.size() * sizeof(int32_t));
        ctx->step_staged = 0;
        stage_upload(ctx, ctx->meta.p, h.data(), h.size() * sizeof(int32_t));

        int32_t* d = ctx->meta.as<int32_t>();
        ctx->dev.past_lens = d;
        ctx->dev.subsequence_begins = d + B;
        ctx->dev.block_indices_begins = d + B + (B + 1);
        ctx->dev.score_window = d + B + 2 * (B + 1);
        ctx->dev.score_offsets = d + 2 * B + 2 * (B + 1);
        ctx->dev.token_seq = d + 2 * B + 3 * (B + 1);
        ctx->dev.gtiles = ctx->dev.token_seq + T;
        ctx->dev.n_gtiles = n_gtiles;
        ctx->dev.B = B;
        ctx->dev.T = T;
        ctx->dev.sliding_window = m->sliding_window;
        ctx->dev.scale = m->scale != 0.0f ? m->scale : 1.0f / std::sqrt((float)ctx->cfg.head_size);
        ctx->B = B;
        ctx->T = T;
        ctx->max_kv = max_kv;
        ctx->total_scores = (int32_t)total_scores;
        ctx->total_block_ids = n_ids;
        ctx->sliding_window = m->sliding_window;
        ctx->scale = ctx->dev.scale;
        ctx->h_past.assign(past, past + B);
        ctx->h_sb.assign(sb, sb + B + 1);
        ctx->h_bib.assign(bib, bib + B + 1);
        // split-K plan: enough waves to fill 256 CUs several times over, at least 256 positions per split
        // (a wave of the shape-generic kernel serves a token tile's rows of up to eight heads of a kv head's group)
        const int64_t rows = std::max<int64_t>(1, (int64_t)n_gtiles * gsh.Hkv * pa::ceil_div(gsh.Hq / gsh.Hkv, gplan.heads));
        const int32_t eff_kv = m->sliding_window > 0 ? std::min(max_kv, m->sliding_window) : max_kv;
        int64_t want = (4096 + rows - 1) / rows;
        int64_t cap = std::max<int64_t>(1, eff_kv / 256);
        ctx->generic_nsplit = (int32_t)std::max<int64_t>(1, std::min<int64_t>(std::min(want, cap), 64));
        ctx->nsplit = ctx->generic_nsplit;
        ctx->h_xseq.clear();
        ctx->h_xseq_of.clear();
        ctx->n_sparse = 0;
        ctx->x_ran = false;
        plan_items(ctx);
        for (auto& c : ctx->table_count) c = -1;  // tables belong to a step
        ctx->step_ready = true;
    });
}

namespace {
// Largest block id of a table + 1 after the check of every id against [0, num_blocks): through the smallest and the
// largest one (a loop without branches, which the compiler turns into vector minima and maxima: 65792 ids take 4 us
// instead of 39).
int64_t checked_bound(const int32_t* ids, int32_t count, int64_t num_blocks) {
    int32_t id_lo = INT32_MAX, id_hi = INT32_MIN;
    for (int32_t i = 0; i < count; ++i) {
        id_lo = std::min(id_lo, ids[i]);
        id_hi = std::max(id_hi, ids[i]);
    }
    PA_REQUIRE(count == 0 || (id_lo >= 0 && id_hi < num_blocks), PA_OUT_OF_BOUNDS, "block index outside the cache");
    return count == 0 ? 0 : (int64_t)id_hi + 1;
}

// Switches the context between one table for all layers and a table per layer.
void shape_tables(pa_ctx* ctx, bool shared) {
    if (!ctx->tables.empty() && shared == ctx->shared_table) return;
    ctx->shared_table = shared;
    const size_t n = shared ? 1 : (size_t)ctx->cfg.num_layers;
    if (ctx->tables.size() != n) {
        HIP_CHECK(hipStreamSynchronize(ctx->stream));
        for (auto& t : ctx->tables) t.release();
        ctx->tables.assign(n, DevBuf());
        ctx->table_ptr.assign(n, nullptr);
        ctx->table_count.assign(n, -1);
        ctx->table_bound.assign(n, 0);
    }
}

// Bytes of a table's upload: the ids, then (u8 decode kernel) the descriptors of its single-token sequences for the
// plan without and the plan with scores.  Sets the descriptors' offsets.
size_t table_upload_bytes(pa_ctx* ctx, int32_t count, size_t* id_bytes, bool* with_descs) {
    *id_bytes = std::max<size_t>(((size_t)count * sizeof(int32_t) + 127) & ~(size_t)127, 128);
    size_t total = *id_bytes;
    *with_descs = decode_u8_step(ctx);
    if (*with_descs)
        for (int w = 0; w < 2; ++w) {
            ctx->desc_off[w] = total;
            total += ctx->h_dec.size() * ctx->dec_plan[w].nsplit * sizeof(pa::DecodeDesc);
        }
    return total;
}

void fill_table_stage(const pa_ctx* ctx, const int32_t* ids, int32_t count, size_t id_bytes, bool with_descs, uint8_t* stage) {
    std::memcpy(stage, ids, (size_t)count * sizeof(int32_t));
    std::memset(stage + (size_t)count * sizeof(int32_t), 0, id_bytes - (size_t)count * sizeof(int32_t));
    if (with_descs) fill_decode_descs(ctx, ids, stage);
}
}  // namespace

int32_t pa_set_block_indices(pa_ctx* ctx, int32_t layer, const int32_t* ids, int32_t count, int64_t num_blocks) {
    if (!ctx) return PA_INVALID_C_PARAM;
    return guarded(ctx, [&] {
        PA_REQUIRE(ctx->step_ready, PA_PARAMETER_MISMATCH, "pa_step_begin has not been called");
        PA_REQUIRE(ids && count >= 0, PA_INVALID_C_PARAM, "block_indices missing");
        PA_REQUIRE(layer >= -1 && layer < ctx->cfg.num_layers, PA_OUT_OF_BOUNDS, "layer out of range");
        PA_REQUIRE(count == ctx->total_block_ids, PA_PARAMETER_MISMATCH,
                   "block_indices length differs from block_indices_begins[B]");
        const int64_t bound = checked_bound(ids, count, num_blocks);
        shape_tables(ctx, layer < 0);
        const size_t idx = layer < 0 ? 0 : (size_t)layer;
        size_t id_bytes;
        bool with_descs;
        const size_t total = table_upload_bytes(ctx, count, &id_bytes, &with_descs);
        HIP_CHECK(hipSetDevice(ctx->cfg.device));
        if (ctx->tables[idx].cap < total) {  // kernels in flight may still read the buffer this would free
            HIP_CHECK(hipStreamSynchronize(ctx->stream));
            ctx->tables[idx].reserve(total);
        }
        uint8_t* stage = stage_piece(ctx, total);
        fill_table_stage(ctx, ids, count, id_bytes, with_descs, stage);
        HIP_CHECK(hipMemcpyAsync(ctx->tables[idx].p, stage, total, hipMemcpyHostToDevice, ctx->stream));
        ctx->table_ptr[idx] = ctx->tables[idx].p;
        ctx->table_count[idx] = count;
        ctx->table_bound[idx] = bound;
    });
}

int32_t pa_set_block_indices_layers(pa_ctx* ctx, int32_t first_layer, int32_t num_layers, const int32_t* const* ids_per_layer,
                                    int32_t count, int64_t num_blocks) {
    if (!ctx) return PA_INVALID_C_PARAM;
    return guarded(ctx, [&] {
        PA_REQUIRE(ctx->step_ready, PA_PARAMETER_MISMATCH, "pa_step_begin has not been called");
        PA_REQUIRE(ids_per_layer && count >= 0 && num_layers > 0, PA_INVALID_C_PARAM, "block_indices missing");
        PA_REQUIRE(first_layer >= 0 && num_layers <= ctx->cfg.num_layers - first_layer, PA_OUT_OF_BOUNDS, "layer out of range");
        for (int32_t l = 0; l < num_layers; ++l) PA_REQUIRE(ids_per_layer[l], PA_INVALID_C_PARAM, "block_indices missing");
        PA_REQUIRE(count == ctx->total_block_ids, PA_PARAMETER_MISMATCH,
                   "block_indices length differs from block_indices_begins[B]");
        shape_tables(ctx, false);
        size_t id_bytes;
        bool with_descs;
        const size_t total = table_upload_bytes(ctx, count, &id_bytes, &with_descs);
        const size_t stride = (total + 255) & ~(size_t)255;
        // One pass of a few host threads over the layers checks every id and fills the layer's piece of the staging
        // area (a table is read once, while it is in the core's cache; memory-bound host work); nothing of the
        // context changes before every layer has passed.
        std::vector<int64_t> bound((size_t)num_layers, 0);
        HIP_CHECK(hipSetDevice(ctx->cfg.device));
        uint8_t* stage = stage_piece(ctx, stride * (size_t)num_layers);
        pa::parallel_items((size_t)num_layers, std::min<size_t>(8, (size_t)num_layers * (size_t)count / 131072 + 1), [&](size_t l) {
            bound[l] = checked_bound(ids_per_layer[l], count, num_blocks);
            fill_table_stage(ctx, ids_per_layer[l], count, id_bytes, with_descs, stage + l * stride);
        });
        if (ctx->table_pool.cap < stride * (size_t)ctx->cfg.num_layers) {
            // kernels in flight may still read the pool this frees; tables that lived in it have to be set again
            HIP_CHECK(hipStreamSynchronize(ctx->stream));
            const uint8_t* old = ctx->table_pool.as<uint8_t>();
            for (size_t i = 0; i < ctx->table_ptr.size(); ++i) {
                const uint8_t* at = static_cast<const uint8_t*>(ctx->table_ptr[i]);
                if (old && at >= old && at < old + ctx->table_pool.cap) {
                    ctx->table_ptr[i] = nullptr;
                    ctx->table_count[i] = -1;
                }
            }
            ctx->table_pool.reserve(stride * (size_t)ctx->cfg.num_layers);
        }
        uint8_t* dst = ctx->table_pool.as<uint8_t>() + (size_t)first_layer * stride;
        HIP_CHECK(hipMemcpyAsync(dst, stage, stride * (size_t)num_layers, hipMemcpyHostToDevice, ctx->stream));
        for (int32_t l = 0; l < num_layers; ++l) {
            const size_t idx = (size_t)(first_layer + l);
            ctx->table_ptr[idx] = dst + (size_t)l * stride;
            ctx->table_count[idx] = count;
            ctx->table_bound[idx] = bound[(size_t)l];
        }
    });
}

int32_t pa_set_xattention(pa_ctx* ctx, const float* thresholds, int32_t block_size, int32_t stride) {
    if (!ctx) return PA_INVALID_C_PARAM;
    return guarded(ctx, [&] {
        PA_REQUIRE(ctx->step_ready, PA_PARAMETER_MISMATCH, "pa_step_begin has not been called");
        const pa_config& c = ctx->cfg;
        const int32_t B = ctx->B;
        const bool had = !ctx->h_xseq.empty();
        ctx->x_ran = false;
        std::vector<pa::XattSeq> seqs;
        std::vector<int32_t> seq_of(B, -1);
        if (thresholds) {
            for (int32_t b = 0; b < B; ++b) {
                PA_REQUIRE(thresholds[b] >= 0.0f && thresholds[b] <= 1.0f, PA_PARAMETER_MISMATCH,
                           "xattention_threshold must lie in [0, 1]");
                const int32_t q_len = ctx->h_sb[b + 1] - ctx->h_sb[b];
                if (thresholds[b] > 0.0f && q_len > 1) {
                    seq_of[b] = (int32_t)seqs.size();
                    pa::XattSeq xs{};
                    xs.b = b;
                    xs.threshold = thresholds[b];
                    seqs.push_back(xs);
                }
            }
        }
        HIP_CHECK(hipSetDevice(c.device));
        if (seqs.empty()) {
            ctx->h_xseq.clear();
            ctx->h_xseq_of.clear();
            if (had) plan_items(ctx);
            return;
        }
        PA_REQUIRE(!ctx->has_alibi, PA_NOT_IMPLEMENTED, "block-sparse prefill is not available with ALiBi slopes");
        PA_REQUIRE(mfma_shape(c) && c.head_size != 96 && c.block_size >= 32, PA_NOT_IMPLEMENTED,
                   "block-sparse prefill needs a block_size of 32 to 256 (a power of two), head_size 64, 128 or 256 and a u8 cache "
                   "or one of the query's type");
        auto pow2 = [](int32_t v) { return v > 0 && (v & (v - 1)) == 0; };
        PA_REQUIRE(pow2(block_size) && block_size >= 32, PA_NOT_IMPLEMENTED,
                   "xattention_block_size must be a power of two, at least 32");
        PA_REQUIRE(pow2(stride) && stride <= 32, PA_NOT_IMPLEMENTED, "xattention_stride must be a power of two, at most 32");
        const int32_t Hq = c.num_heads;
        int64_t logit_off = 0, sum_off = 0, mask_off = 0;
        std::vector<pa::XattTile> tiles;
        int32_t max_nqs = 0, max_nqb = 0, max_nkb = 0;
        for (size_t x = 0; x < seqs.size(); ++x) {
            pa::XattSeq& xs = seqs[x];
            const int32_t past = ctx->h_past[xs.b], kv_len = past + ctx->h_sb[xs.b + 1] - ctx->h_sb[xs.b];
            xs.qb0 = past / block_size;
            xs.nkb = (kv_len - 1) / block_size + 1;
            xs.nqb = xs.nkb - xs.qb0;
            xs.words = (xs.nkb + 31) / 32;
            xs.qs0 = past / stride;
            xs.nks = (kv_len - 1) / stride + 1;
            xs.nqs = xs.nks - xs.qs0;
            xs.ld = (xs.nks + 127) & ~127;
            PA_REQUIRE(xs.nkb <= 2048, PA_NOT_IMPLEMENTED, "block-sparse prefill: more than 2048 key blocks in a sequence");
            const int32_t rows = (xs.nqs + 31) & ~31;
            xs.logit_off = logit_off;
            xs.sum_off = sum_off;
            xs.mask_off = mask_off;
            logit_off += (int64_t)Hq * rows * xs.ld;
            sum_off += (int64_t)Hq * xs.nqb * xs.nkb;
            mask_off += (int64_t)Hq * xs.nqb * xs.words;
            for (int32_t it = 0; it < rows / 32; ++it) {
                const int32_t last = xs.qs0 + std::min(32 * it + 31, xs.nqs - 1);  // last strided query group of the tile
                for (int32_t jc = 0; pa::XATT_KEY_TILE * jc <= last; ++jc) tiles.push_back({(int32_t)x, it, jc, 0});
            }
            max_nqs = std::max(max_nqs, xs.nqs);
            max_nqb = std::max(max_nqb, xs.nqb);
            max_nkb = std::max(max_nkb, xs.nkb);
        }
        PA_REQUIRE(logit_off * 4 <= ((int64_t)4 << 30), PA_NOT_ALLOCATED,
                   "block-sparse prefill: the strided logits of this step exceed 4 GiB (larger stride or shorter chunks)");
        // (pa_step_begin has waited for the previous step's kernels, which read the old plan; the copies are queued)
        const size_t seq_bytes = seqs.size() * sizeof(pa::XattSeq), tile_bytes = tiles.size() * sizeof(pa::XattTile);
        ctx->x_tiles_off = seq_bytes;
        ctx->x_seq_of_off = seq_bytes + tile_bytes;
        ctx->x_plan.reserve(seq_bytes + tile_bytes + (size_t)B * sizeof(int32_t));
        uint8_t* d = static_cast<uint8_t*>(ctx->x_plan.p);
        stage_upload(ctx, d, seqs.data(), seq_bytes);
        stage_upload(ctx, d + seq_bytes, tiles.data(), tile_bytes);
        stage_upload(ctx, d + seq_bytes + tile_bytes, seq_of.data(), (size_t)B * sizeof(int32_t));
        ctx->x_logits.reserve((size_t)logit_off * sizeof(float));
        ctx->x_sums.reserve((size_t)sum_off * sizeof(float));
        ctx->x_mask.reserve((size_t)mask_off * sizeof(uint32_t));
        ctx->h_xseq = seqs;
        ctx->h_xseq_of = seq_of;
        ctx->xatt_block = block_size;
        ctx->xatt_stride = stride;
        ctx->x_ntiles = (int32_t)tiles.size();
        ctx->x_max_nqs = max_nqs;
        ctx->x_max_nqb = max_nqb;
        ctx->x_max_nkb = max_nkb;
        plan_items(ctx);
        ctx->x_item_keep.reserve((size_t)std::max(1, ctx->n_sparse) * c.num_kv_heads * ctx->x_keep_words * sizeof(int32_t));
    });
}

int32_t pa_xattention_shape(const pa_ctx* ctx, int32_t sequence, int32_t* first_query_block, int32_t* num_query_blocks,
                            int32_t* num_key_blocks) {
    if (!ctx || !first_query_block || !num_query_blocks || !num_key_blocks) return PA_INVALID_C_PARAM;
    if (!ctx->step_ready || sequence < 0 || sequence >= ctx->B) return PA_OUT_OF_BOUNDS;
    const int x = xatt_seq_index(ctx, sequence);
    *first_query_block = x < 0 ? 0 : ctx->h_xseq[x].qb0;
    *num_query_blocks = x < 0 ? 0 : ctx->h_xseq[x].nqb;
    *num_key_blocks = x < 0 ? 0 : ctx->h_xseq[x].nkb;
    return PA_OK;
}

int32_t pa_xattention_block_sums(pa_ctx* ctx, int32_t sequence, float* sums) {
    if (!ctx) return PA_INVALID_C_PARAM;
    return guarded(ctx, [&] {
        PA_REQUIRE(ctx->step_ready && sequence >= 0 && sequence < ctx->B, PA_OUT_OF_BOUNDS, "no such sequence in the step");
        const int x = xatt_seq_index(ctx, sequence);
        PA_REQUIRE(x >= 0 && sums, PA_PARAMETER_MISMATCH, "the sequence is not block-sparse in this step");
        PA_REQUIRE(ctx->x_ran, PA_PARAMETER_MISMATCH, "no layer call of this step has run yet");
        const pa::XattSeq& xs = ctx->h_xseq[x];
        HIP_CHECK(hipSetDevice(ctx->cfg.device));
        HIP_CHECK(hipStreamSynchronize(ctx->stream));
        HIP_CHECK(hipMemcpy(sums, ctx->x_sums.as<float>() + xs.sum_off,
                            (size_t)ctx->cfg.num_heads * xs.nqb * xs.nkb * sizeof(float), hipMemcpyDeviceToHost));
    });
}

int32_t pa_xattention_retained(pa_ctx* ctx, int32_t sequence, uint8_t* retained) {
    if (!ctx) return PA_INVALID_C_PARAM;
    return guarded(ctx, [&] {
        PA_REQUIRE(ctx->step_ready && sequence >= 0 && sequence < ctx->B, PA_OUT_OF_BOUNDS, "no such sequence in the step");
        const int x = xatt_seq_index(ctx, sequence);
        PA_REQUIRE(x >= 0 && retained, PA_PARAMETER_MISMATCH, "the sequence is not block-sparse in this step");
        PA_REQUIRE(ctx->x_ran, PA_PARAMETER_MISMATCH, "no layer call of this step has run yet");
        const pa::XattSeq& xs = ctx->h_xseq[x];
        const size_t rows = (size_t)ctx->cfg.num_heads * xs.nqb;
        std::vector<uint32_t> words(rows * xs.words);
        HIP_CHECK(hipSetDevice(ctx->cfg.device));
        HIP_CHECK(hipStreamSynchronize(ctx->stream));
        HIP_CHECK(hipMemcpy(words.data(), ctx->x_mask.as<uint32_t>() + xs.mask_off, words.size() * sizeof(uint32_t),
                            hipMemcpyDeviceToHost));
        for (size_t r = 0; r < rows; ++r)
            for (int32_t J = 0; J < xs.nkb; ++J)
                retained[r * xs.nkb + J] = (words[r * xs.words + J / 32] >> (J % 32)) & 1u;
    });
}

float pa_xattention_threshold(float configured_threshold, uint64_t num_last_dense_tokens_in_prefill, uint64_t prompt_len,
                              uint64_t num_processed_tokens, uint64_t num_scheduled_tokens, int32_t can_generate_tokens) {
    if (can_generate_tokens && num_scheduled_tokens == 1) return 0.0f;  // generation phase
    const uint64_t after = num_processed_tokens + num_scheduled_tokens;
    if (after < prompt_len && prompt_len - after < num_last_dense_tokens_in_prefill) return 0.0f;  // dense tail
    return configured_threshold;
}

int32_t pa_kv_append(pa_ctx* ctx, int32_t layer, const pa_layer_io* io) {
    if (!ctx) return PA_INVALID_C_PARAM;
    return guarded(ctx, [&] {
        HIP_CHECK(hipSetDevice(ctx->cfg.device));
        do_kv_append(ctx, layer, io);
    });
}

int32_t pa_attention(pa_ctx* ctx, int32_t layer, const pa_layer_io* io) {
    if (!ctx) return PA_INVALID_C_PARAM;
    return guarded(ctx, [&] {
        HIP_CHECK(hipSetDevice(ctx->cfg.device));
        do_attention(ctx, layer, io);
    });
}

int32_t pa_attention_static(pa_ctx* ctx, int32_t layer, const pa_layer_io* io) {
    if (!ctx) return PA_INVALID_C_PARAM;
    return guarded(ctx, [&] {
        HIP_CHECK(hipSetDevice(ctx->cfg.device));
        do_attention(ctx, layer, io, true);
    });
}

int32_t pa_forward(pa_ctx* ctx, int32_t layer, const pa_layer_io* io) {
    if (!ctx) return PA_INVALID_C_PARAM;
    return guarded(ctx, [&] {
        HIP_CHECK(hipSetDevice(ctx->cfg.device));
        // a step of single-token sequences that all go to one of the decode kernels: it appends the new rows itself
        const bool fuse = ctx->step_ready &&
                          ((decode_u8_shape(ctx) && (int32_t)ctx->h_dec.size() == ctx->B) ||
                           (mfma_shape(ctx) && decode16_shape(ctx) && (int32_t)ctx->h_dec16.size() == ctx->B &&
                            ctx->n_sparse == 0 && ctx->n_single == ctx->n_items));
        if (fuse) check_io(ctx, layer, io, true, false);
        else do_kv_append(ctx, layer, io);
        do_attention(ctx, layer, io, false, fuse);
    });
}

int32_t pa_synchronize(pa_ctx* ctx) {
    if (!ctx) return PA_INVALID_C_PARAM;
    return guarded(ctx, [&] {
        HIP_CHECK(hipSetDevice(ctx->cfg.device));
        HIP_CHECK(hipStreamSynchronize(ctx->stream));
    });
}

int32_t pa_get_num_splits(const pa_ctx* ctx) { return ctx ? ctx->nsplit : 0; }

int32_t pa_set_profiling(pa_ctx* ctx, int32_t enable) {
    if (!ctx) return PA_INVALID_C_PARAM;
    return guarded(ctx, [&] {
        HIP_CHECK(hipSetDevice(ctx->cfg.device));
        if (enable && !ctx->ev0) {
            HIP_CHECK(hipEventCreate(&ctx->ev0));
            HIP_CHECK(hipEventCreate(&ctx->ev1));
        }
        ctx->profiling = enable != 0;
        ctx->timed = false;
    });
}

int32_t pa_last_kernel_ms(pa_ctx* ctx, float* ms) {
    if (!ctx || !ms) return PA_INVALID_C_PARAM;
    return guarded(ctx, [&] {
        PA_REQUIRE(ctx->timed, PA_PARAMETER_MISMATCH, "no attention call has been timed (pa_set_profiling)");
        HIP_CHECK(hipSetDevice(ctx->cfg.device));
        HIP_CHECK(hipEventSynchronize(ctx->ev1));
        HIP_CHECK(hipEventElapsedTime(ms, ctx->ev0, ctx->ev1));
    });
}

// ------------------------------------------------------------------------------------ step packing
int32_t pa_trishape_skipped_blocks(uint64_t block_size, uint64_t num_last_dense, uint64_t retained_start,
                                   uint64_t retained_recent, uint64_t prompt_len, uint64_t num_processed,
                                   uint64_t num_scheduled, uint64_t num_cached, uint64_t* first_skipped,
                                   uint64_t* num_skipped) {
    return guarded<NoObj>(nullptr, [&] {
        PA_REQUIRE(first_skipped && num_skipped, PA_INVALID_C_PARAM, "null output");
        PA_REQUIRE(block_size > 0, PA_PARAMETER_MISMATCH, "block_size must be positive");
        PA_REQUIRE(retained_start % block_size == 0 && retained_recent % block_size == 0, PA_PARAMETER_MISMATCH,
                   "retained start / recent areas must be multiples of the block size");
        const uint64_t after = num_processed + num_scheduled;
        PA_REQUIRE(prompt_len >= after, PA_PARAMETER_MISMATCH, "the chunk runs past the prompt");
        *first_skipped = retained_start / block_size;
        *num_skipped = 0;
        if (prompt_len - after < num_last_dense) return;  // dense phase
        const uint64_t full = num_cached / block_size;
        const uint64_t retained = retained_start / block_size + retained_recent / block_size;
        if (full > retained) *num_skipped = full - retained;
    });
}

int32_t pa_rotation_trig_lut(int32_t block_size, int32_t max_blocks, int32_t head_size, double rope_theta, float* lut) {
    return guarded<NoObj>(nullptr, [&] {
        PA_REQUIRE(lut, PA_INVALID_C_PARAM, "lut is null");
        PA_REQUIRE(block_size > 0 && max_blocks >= 0 && head_size > 0 && head_size % 2 == 0, PA_PARAMETER_MISMATCH,
                   "block_size and head_size must be positive, head_size even");
        PA_REQUIRE(rope_theta > 0, PA_PARAMETER_MISMATCH, "rope_theta must be positive");
        const int32_t nf = head_size / 2;
        for (int32_t i = 0; i < max_blocks; ++i)
            for (int32_t j = 0; j < nf; ++j) {
                const double exponent = -static_cast<double>(2 * j) / head_size;
                const double angle = static_cast<double>((int64_t)i * block_size) * std::pow(rope_theta, exponent);
                lut[(size_t)i * head_size + j] = static_cast<float>(std::cos(angle));
                lut[(size_t)i * head_size + nf + j] = static_cast<float>(-std::sin(angle));
            }
    });
}

int32_t pa_rotation_data(const int64_t* evicted, int32_t num_evicted, int64_t num_blocks_before, int32_t block_size,
                         int32_t max_blocks, int32_t* logical_block_idx, int32_t* rotation_delta_tokens,
                         int32_t capacity, int32_t* count) {
    return guarded<NoObj>(nullptr, [&] {
        PA_REQUIRE(count && num_evicted >= 0 && (evicted || num_evicted == 0), PA_INVALID_C_PARAM, "null argument");
        PA_REQUIRE(block_size > 0 && num_blocks_before >= 0 && capacity >= 0, PA_PARAMETER_MISMATCH, "bad sizes");
        PA_REQUIRE((logical_block_idx && rotation_delta_tokens) || capacity == 0, PA_INVALID_C_PARAM, "null output");
        *count = 0;
        if (num_evicted == 0) return;
        std::vector<int64_t> ev(evicted, evicted + num_evicted);
        std::sort(ev.begin(), ev.end());
        ev.erase(std::unique(ev.begin(), ev.end()), ev.end());
        PA_REQUIRE(ev.front() >= 0 && ev.back() < num_blocks_before, PA_OUT_OF_BOUNDS,
                   "evicted block index beyond the blocks occupied before eviction");
        size_t next = 0;
        int64_t shift = 0;
        int32_t n = 0;
        for (int64_t b = 0; b < num_blocks_before; ++b) {
            if (next < ev.size() && ev[next] == b) {
                ++next;
                ++shift;
            } else if (shift != 0) {
                PA_REQUIRE(shift <= max_blocks, PA_OUT_OF_BOUNDS, "rotation delta larger than LUT size");
                if (n < capacity) {
                    logical_block_idx[n] = (int32_t)(b - shift);
                    rotation_delta_tokens[n] = (int32_t)(shift * block_size);
                }
                ++n;
            }
        }
        *count = n;
    });
}

int32_t pa_set_alibi_slopes(pa_ctx* ctx, const float* slopes, int32_t count) {
    if (!ctx) return PA_INVALID_C_PARAM;
    return guarded(ctx, [&] {
        PA_REQUIRE(count == 0 || (slopes && count == ctx->cfg.num_heads), PA_PARAMETER_MISMATCH,
                   "alibi_slopes must be empty or hold one slope per query head");
        bool any = false;
        for (int32_t h = 0; h < count; ++h) {
            PA_REQUIRE(std::isfinite(slopes[h]), PA_PARAMETER_MISMATCH, "alibi_slopes must be finite");
            any = any || slopes[h] != 0.0f;
        }
        HIP_CHECK(hipSetDevice(ctx->cfg.device));
        HIP_CHECK(hipStreamSynchronize(ctx->stream));  // earlier launches may still read the old slopes
        if (any) {
            const size_t bytes = (size_t)count * sizeof(float);
            ctx->alibi.reserve(bytes);
            HIP_CHECK(hipMemcpyAsync(ctx->alibi.p, slopes, bytes, hipMemcpyHostToDevice, ctx->stream));
            HIP_CHECK(hipStreamSynchronize(ctx->stream));  // `slopes` is the caller's, pageable
        }
        // the step's plan depends on which kernels serve it: a step that has begun has to begin again
        if (any != ctx->has_alibi) ctx->step_ready = false;
        ctx->has_alibi = any;
    });
}

int32_t pa_set_rotation_trig_lut(pa_ctx* ctx, const float* lut, int32_t rows) {
    if (!ctx) return PA_INVALID_C_PARAM;
    return guarded(ctx, [&] {
        PA_REQUIRE(lut && rows > 0, PA_INVALID_C_PARAM, "trig table missing");
        HIP_CHECK(hipSetDevice(ctx->cfg.device));
        HIP_CHECK(hipStreamSynchronize(ctx->stream));  // an earlier rotation may still read the old table
        const size_t bytes = (size_t)rows * ctx->cfg.head_size * sizeof(float);
        ctx->trig_lut.reserve(bytes);
        HIP_CHECK(hipMemcpyAsync(ctx->trig_lut.p, lut, bytes, hipMemcpyHostToDevice, ctx->stream));
        HIP_CHECK(hipStreamSynchronize(ctx->stream));  // `lut` is the caller's, pageable
        ctx->trig_rows = rows;
    });
}

int32_t pa_rotate_cache(pa_ctx* ctx, void* key_cache, int64_t num_blocks, const int32_t* rotated_block_indices,
                        int32_t num_rotated, const int32_t* rotation_deltas, int32_t deltas_per_block) {
    if (!ctx) return PA_INVALID_C_PARAM;
    return guarded(ctx, [&] {
        const pa_config& c = ctx->cfg;
        PA_REQUIRE(num_rotated >= 0, PA_INVALID_C_PARAM, "negative block count");
        if (num_rotated == 0) return;
        PA_REQUIRE(key_cache && rotated_block_indices && rotation_deltas, PA_INVALID_C_PARAM, "null argument");
        PA_REQUIRE((reinterpret_cast<uintptr_t>(key_cache) & 15) == 0, PA_INVALID_C_PARAM,
                   "the key cache must start at a multiple of 16 bytes");
        PA_REQUIRE(ctx->trig_rows > 0, PA_NOT_ALLOCATED, "pa_set_rotation_trig_lut has not been called");
        PA_REQUIRE(c.kv_cache_dtype != PA_U4, PA_NOT_IMPLEMENTED, "cache rotation runs over u8, f16 and bf16 key caches");
        PA_REQUIRE(deltas_per_block == 1 || deltas_per_block == c.block_size, PA_PARAMETER_MISMATCH,
                   "rotation_deltas must hold 1 or block_size entries per block");
        for (int32_t i = 0; i < num_rotated; ++i)
            PA_REQUIRE(rotated_block_indices[i] >= 0 && rotated_block_indices[i] < num_blocks, PA_OUT_OF_BOUNDS,
                       "rotated block index outside the cache");
        const size_t n_delta = (size_t)num_rotated * deltas_per_block;
        for (size_t i = 0; i < n_delta; ++i)
            PA_REQUIRE(rotation_deltas[i] >= 0 && rotation_deltas[i] < ctx->trig_rows, PA_OUT_OF_BOUNDS,
                       "rotation delta beyond the trig table");
        HIP_CHECK(hipSetDevice(c.device));
        // (the previous call's kernel may still read the arguments: the copies below are ordered behind it on the
        // stream, and a buffer that has to grow is freed by a call that waits for the device)
        ctx->rot_args.reserve((num_rotated + n_delta) * sizeof(int32_t));
        int32_t* d_idx = ctx->rot_args.as<int32_t>();
        int32_t* d_delta = d_idx + num_rotated;
        stage_upload(ctx, d_idx, rotated_block_indices, num_rotated * sizeof(int32_t));
        stage_upload(ctx, d_delta, rotation_deltas, n_delta * sizeof(int32_t));
        HIP_CHECK(pa::launch_rotate(ctx->stream, key_cache, c.kv_cache_dtype, shape_of(c), d_idx, d_delta,
                                    deltas_per_block, num_rotated, ctx->trig_lut.as<float>()));
    });
}

int32_t pa_adaptive_rkv_diversity(pa_ctx* ctx, int32_t layer, const void* key_cache, int64_t num_blocks,
                                  int32_t start_size, const int32_t* evictable_sizes, float* diversity,
                                  int64_t capacity, int64_t* offsets) {
    if (!ctx) return PA_INVALID_C_PARAM;
    return guarded(ctx, [&] {
        const pa_config& c = ctx->cfg;
        PA_REQUIRE(ctx->step_ready, PA_PARAMETER_MISMATCH, "pa_step_begin has not been called");
        PA_REQUIRE(evictable_sizes, PA_INVALID_C_PARAM, "adaptive_rkv_evictable_sizes missing");
        PA_REQUIRE(layer >= 0 && layer < c.num_layers, PA_OUT_OF_BOUNDS, "layer out of range");
        // the matrix-core kernels' shapes; everything else runs on the vector unit
        const bool tuned = c.block_size == 32 && (c.head_size == 64 || c.head_size == 96 || c.head_size == 128 || c.head_size == 256) &&
                           c.kv_cache_dtype != PA_U4;
        PA_REQUIRE(start_size >= 0 && start_size % c.block_size == 0, PA_PARAMETER_MISMATCH,
                   "adaptive_rkv_start_size must be a non-negative multiple of the block size");
        const size_t tidx = ctx->shared_table ? 0 : (size_t)layer;
        PA_REQUIRE(tidx < ctx->tables.size() && ctx->table_count[tidx] == ctx->total_block_ids, PA_PARAMETER_MISMATCH,
                   "pa_set_block_indices has not been called for this layer in this step");
        std::vector<pa::RkvDivSeq> seqs;
        int64_t out_total = 0, tok_total = 0;
        int32_t ev_max = 0;
        if (offsets) offsets[0] = 0;
        for (int32_t b = 0; b < ctx->B; ++b) {
            const int32_t ev = evictable_sizes[b];
            PA_REQUIRE(ev >= 0 && ev % c.block_size == 0, PA_PARAMETER_MISMATCH,
                       "adaptive_rkv_evictable_sizes must hold non-negative multiples of the block size");
            if (ev > 0) {
                const int64_t kv_len = (int64_t)ctx->h_past[b] + (ctx->h_sb[b + 1] - ctx->h_sb[b]);
                PA_REQUIRE((int64_t)start_size + ev <= kv_len, PA_OUT_OF_BOUNDS,
                           "start and evictable areas reach beyond the sequence's keys");
                PA_REQUIRE((start_size + ev) / c.block_size <= ctx->h_bib[b + 1] - ctx->h_bib[b], PA_OUT_OF_BOUNDS,
                           "start and evictable areas reach beyond the sequence's block table");
                seqs.push_back(pa::RkvDivSeq{ctx->h_bib[b], start_size / c.block_size, ev, (int32_t)tok_total, out_total});
                out_total += (int64_t)(ev / c.block_size) * ev;
                tok_total += ev;
                ev_max = std::max(ev_max, ev);
                PA_REQUIRE(tok_total <= INT32_MAX / 4, PA_OUT_OF_BOUNDS, "evictable areas too large for one call");
            }
            if (offsets) offsets[b + 1] = out_total;
        }
        if (seqs.empty()) return;
        PA_REQUIRE(key_cache && diversity, PA_INVALID_C_PARAM, "null argument");
        PA_REQUIRE((reinterpret_cast<uintptr_t>(key_cache) & 15) == 0 && (reinterpret_cast<uintptr_t>(diversity) & 3) == 0,
                   PA_INVALID_C_PARAM, "the key cache must start at a multiple of 16 bytes, the output at a multiple of 4");
        PA_REQUIRE(out_total <= capacity, PA_OUT_OF_BOUNDS, "diversity output holds fewer values than the areas need");
        // the areas' blocks must exist in the cache handed over now (the table was checked against the num_blocks of
        // its own call)
        PA_REQUIRE(num_blocks >= ctx->table_bound[tidx] && num_blocks > 0, PA_OUT_OF_BOUNDS,
                   "the key cache holds fewer blocks than the block table of this layer refers to");
        HIP_CHECK(hipSetDevice(c.device));
        // (the previous call's kernels may still read the sequence list and the work buffers: this call's copy and
        // kernels are ordered behind them on the stream, and a buffer that has to grow is freed by a call that waits)
        const int chunks = pa::rkv_diversity_chunks(ev_max);
        ctx->div_seqs.reserve(seqs.size() * sizeof(pa::RkvDivSeq));
        ctx->div_stats.reserve((size_t)c.num_kv_heads * tok_total * sizeof(float4));
        ctx->div_mean.reserve((size_t)c.num_kv_heads * tok_total * sizeof(float));
        ctx->div_colsum.reserve(seqs.size() * c.num_kv_heads * (chunks + 1) * c.head_size * sizeof(float));
        stage_upload(ctx, ctx->div_seqs.p, seqs.data(), seqs.size() * sizeof(pa::RkvDivSeq));
        pa::RkvDivArgs a{};
        a.key_cache = static_cast<const uint8_t*>(key_cache);
        a.block_indices = static_cast<const int32_t*>(ctx->table_ptr[tidx]);
        a.seqs = ctx->div_seqs.as<pa::RkvDivSeq>();
        a.stats = ctx->div_stats.as<float4>();
        a.mean = ctx->div_mean.as<float>();
        a.colsum = ctx->div_colsum.as<float>();
        a.out = diversity;
        a.Hkv = c.num_kv_heads;
        a.total_tok = (int32_t)tok_total;
        a.chunks_max = chunks;
        if (tuned)
            HIP_CHECK(pa::launch_rkv_diversity(ctx->stream, a, c.kv_cache_dtype, c.head_size, c.block_size, (int)seqs.size(), ev_max));
        else
            HIP_CHECK(pa::launch_rkv_diversity_generic(ctx->stream, a, c.kv_cache_dtype, c.head_size, c.block_size, (int)seqs.size(), ev_max));
    });
}

int32_t pa_pack_step(int32_t B, const int64_t* processed, const int64_t* evicted, const int64_t* skipped_blocks,
                     const int64_t* scheduled, const int64_t* num_blocks, int32_t block_size, int32_t* past_lens,
                     int32_t* subsequence_begins, int32_t* block_indices_begins, int32_t* max_context_len) {
    return guarded<NoObj>(nullptr, [&] {
        PA_REQUIRE(B >= 0 && processed && evicted && scheduled && num_blocks && past_lens && subsequence_begins &&
                       block_indices_begins && max_context_len,
                   PA_INVALID_C_PARAM, "null argument");
        PA_REQUIRE(block_size > 0, PA_PARAMETER_MISMATCH, "block_size must be positive");
        int64_t tokens = 0, blocks = 0, longest = 0;
        subsequence_begins[0] = 0;
        block_indices_begins[0] = 0;
        for (int32_t b = 0; b < B; ++b) {
            const int64_t skip = skipped_blocks ? skipped_blocks[b] : 0;
            PA_REQUIRE(num_blocks[b] >= skip, PA_PARAMETER_MISMATCH, "more skipped blocks than blocks");
            const int64_t past = processed[b] - evicted[b] - skip * block_size;
            PA_REQUIRE(past >= 0 && past <= INT32_MAX, PA_OUT_OF_BOUNDS, "past length out of range");
            tokens += scheduled[b];
            blocks += num_blocks[b] - skip;
            PA_REQUIRE(tokens <= INT32_MAX && blocks <= INT32_MAX, PA_OUT_OF_BOUNDS, "step too large for int32");
            past_lens[b] = (int32_t)past;
            subsequence_begins[b + 1] = (int32_t)tokens;
            block_indices_begins[b + 1] = (int32_t)blocks;
            longest = std::max(longest, processed[b] + scheduled[b]);
        }
        PA_REQUIRE(longest <= INT32_MAX, PA_OUT_OF_BOUNDS, "context length overflows int32");
        *max_context_len = (int32_t)longest;
    });
}

uint64_t pa_snapkv_num_scores(uint64_t window, uint64_t prompt_len, uint64_t scheduled, uint64_t processed) {
    if (window == 0) return scheduled;
    const uint64_t first_scored = window > prompt_len ? 0 : prompt_len - window;
    const uint64_t after = processed + scheduled;
    if (after <= first_scored) return 0;
    return processed > first_scored ? scheduled : after - first_scored;
}

// ------------------------------------------------------------------------------------ KV cache tensors
namespace {

hipMemAllocationProp device_memory_prop(int device) {
    hipMemAllocationProp prop{};
    prop.type = hipMemAllocationTypePinned;
    prop.location.type = hipMemLocationTypeDevice;
    prop.location.id = device;
    return prop;
}

// Unmaps and releases the chunks of every tensor from index `from[t]` on.
void drop_chunks(pa_kv_cache* c, const std::vector<size_t>& from) {
    for (size_t t = 0; t < c->chunks.size(); ++t) {
        auto& list = c->chunks[t];
        while (list.size() > from[t]) {
            const pa_kv_cache::Chunk& ch = list.back();
            (void)hipMemUnmap(static_cast<uint8_t*>(c->tensor(t)) + ch.offset, ch.bytes);
            (void)hipMemRelease(ch.handle);
            list.pop_back();
        }
    }
}

void destroy_kv_cache(pa_kv_cache* c) {
    (void)hipSetDevice(c->cfg.device);
    (void)hipDeviceSynchronize();
    drop_chunks(c, std::vector<size_t>(c->chunks.size(), 0));
    for (size_t t = 0; t < 2 * c->key.size(); ++t)
        if (c->tensor(t)) (void)hipMemAddressFree(c->tensor(t), c->reserved[t]);
    c->base_table.release();
    c->pairs.release();
    delete c;
}

}  // namespace

namespace {
// The tensors of a cache from one description per layer (key and value side of each).
void create_kv_cache(int32_t device, void* stream, const pa_kv_layer_desc* layers, int32_t num_layers, pa_kv_cache** out) {
    PA_REQUIRE(out, PA_INVALID_C_PARAM, "out is null");
    *out = nullptr;
    PA_REQUIRE(layers && num_layers > 0, PA_INVALID_C_PARAM, "layer descriptions missing");
    int ndev = 0;
    HIP_CHECK(hipGetDeviceCount(&ndev));
    PA_REQUIRE(device >= 0 && device < ndev, PA_OUT_OF_BOUNDS, "no such HIP device");
    HIP_CHECK(hipSetDevice(device));
    pa_kv_cache* c = new pa_kv_cache();
    c->cfg.device = device;
    c->cfg.stream = stream;
    c->cfg.num_layers = num_layers;
    const size_t n_tensors = 2 * (size_t)num_layers;
    c->key.assign(num_layers, nullptr);
    c->value.assign(num_layers, nullptr);
    c->chunks.assign(n_tensors, {});
    c->block_bytes.assign(n_tensors, 0);
    c->reserved.assign(n_tensors, 0);
    c->mapped.assign(n_tensors, 0);
    try {
        for (size_t t = 0; t < n_tensors; ++t) {
            const pa_kv_tensor_desc& d = (t & 1) ? layers[t >> 1].value : layers[t >> 1].key;
            PA_REQUIRE(d.num_kv_heads > 0 && d.block_size > 0 && d.head_size > 0, PA_PARAMETER_MISMATCH,
                       "kv heads, block size and head size of a cache tensor must be positive");
            PA_REQUIRE(d.dtype == PA_F16 || d.dtype == PA_BF16 || d.dtype == PA_U8 || d.dtype == PA_U4, PA_PARAMETER_MISMATCH,
                       "a cache tensor's type must be PA_U8, PA_U4, PA_F16 or PA_BF16");
            PA_REQUIRE(d.dtype != PA_U4 || d.head_size % 2 == 0, PA_PARAMETER_MISMATCH, "u4 rows hold an even number of elements");
            c->block_bytes[t] = (uint64_t)d.num_kv_heads * d.block_size * pa::row_bytes(d.head_size, d.dtype);
            PA_REQUIRE(c->block_bytes[t] % 16 == 0, PA_NOT_IMPLEMENTED, "a block of one tensor must be a multiple of 16 bytes");
        }
        const hipMemAllocationProp prop = device_memory_prop(device);
        size_t reported = 0;
        HIP_CHECK(hipMemGetAllocationGranularity(&reported, &prop, hipMemAllocationGranularityRecommended));
        PA_REQUIRE(reported > 0, PA_GENERAL_ERROR, "the device reports no allocation granularity");
        // address space for as much as the device could ever hold, shared between the tensors in proportion to their
        // block sizes
        size_t free_b = 0, total_b = 0;
        HIP_CHECK(hipMemGetInfo(&free_b, &total_b));
        // A tensor's memory is mapped in pieces of one size, each at a multiple of that size: on this device pieces
        // of differing sizes behind one another were refused now and then (hipMemSetAccess: invalid argument), and so
        // were pieces at offsets aligned only to the 4 KiB the runtime reports; equal pieces never were.  The size is
        // a power of two near 1/1024 of the tensor's address range, between 2 MiB and 64 MiB: at most about a
        // thousand pieces per tensor (each costs about 60 us to create and map), at most one piece per tensor unused.
        size_t piece = (size_t)2 << 20;
        while (piece < ((size_t)64 << 20) && piece < total_b / n_tensors / 1024) piece *= 2;
        PA_REQUIRE(piece % reported == 0, PA_GENERAL_ERROR, "unexpected allocation granularity");
        c->granularity = piece;
        const uint64_t all = c->all_block_bytes();
        for (size_t t = 0; t < n_tensors; ++t) {
            const size_t share = (size_t)((double)total_b * ((double)c->block_bytes[t] / (double)all));
            c->reserved[t] = (share + piece - 1) / piece * piece;
            HIP_CHECK(hipMemAddressReserve(&c->tensor(t), c->reserved[t], c->granularity, nullptr, 0));
        }
        // for the copy kernel: the base addresses, then the block sizes
        std::vector<uint64_t> table(2 * n_tensors);
        for (size_t t = 0; t < n_tensors; ++t) {
            table[t] = (uint64_t)(uintptr_t)c->tensor(t);
            table[n_tensors + t] = c->block_bytes[t];
        }
        c->base_table.reserve(table.size() * sizeof(uint64_t));
        HIP_CHECK(hipMemcpy(c->base_table.p, table.data(), table.size() * sizeof(uint64_t), hipMemcpyHostToDevice));
    } catch (...) {
        destroy_kv_cache(c);
        throw;
    }
    *out = c;
}
}  // namespace

int32_t pa_kv_cache_create(const pa_config* cfg, pa_kv_cache** out) {
    return guarded<NoObj>(nullptr, [&] {
        PA_REQUIRE(out, PA_INVALID_C_PARAM, "out is null");
        *out = nullptr;
        check_config(cfg);
        pa_kv_layer_desc one{};
        one.key = pa_kv_tensor_desc{cfg->num_kv_heads, cfg->block_size, cfg->head_size, cfg->kv_cache_dtype};
        one.value = pa_kv_tensor_desc{cfg->num_kv_heads, cfg->block_size, v_head(*cfg), v_dtype(*cfg)};
        const std::vector<pa_kv_layer_desc> layers((size_t)cfg->num_layers, one);
        create_kv_cache(cfg->device, cfg->stream, layers.data(), cfg->num_layers, out);
    });
}

int32_t pa_kv_cache_create_layers(int32_t device, void* stream, const pa_kv_layer_desc* layers, int32_t num_layers,
                                  pa_kv_cache** out) {
    return guarded<NoObj>(nullptr, [&] { create_kv_cache(device, stream, layers, num_layers, out); });
}

void pa_kv_cache_destroy(pa_kv_cache* c) {
    if (c) destroy_kv_cache(c);
}

const char* pa_kv_cache_last_error(const pa_kv_cache* c) { return c ? c->error.c_str() : g_last_error.c_str(); }

uint64_t pa_kv_cache_block_bytes(const pa_kv_cache* c) { return c ? c->all_block_bytes() : 0; }

uint64_t pa_kv_cache_num_blocks(const pa_kv_cache* c) { return c ? c->num_blocks : 0; }

int32_t pa_kv_cache_allocate(pa_kv_cache* c, uint64_t num_kv_blocks) {
    if (!c) return PA_INVALID_C_PARAM;
    return guarded(c, [&] {
        if (c->num_blocks >= num_kv_blocks) return;
        HIP_CHECK(hipSetDevice(c->cfg.device));
        hipStream_t s = static_cast<hipStream_t>(c->cfg.stream);
        const char* too_large = "Requested KV-cache size is larger than available memory size on the system.";
        const size_t n_tensors = c->chunks.size(), piece = c->granularity;
        // what every tensor needs mapped, and how many new pieces that is
        std::vector<size_t> need(n_tensors), first_new(n_tensors + 1, 0);
        for (size_t t = 0; t < n_tensors; ++t) {
            PA_REQUIRE(num_kv_blocks <= c->reserved[t] / c->block_bytes[t], PA_NOT_ALLOCATED, too_large);
            need[t] = ((size_t)(num_kv_blocks * c->block_bytes[t]) + piece - 1) / piece * piece;
            first_new[t + 1] = first_new[t] + (need[t] > c->mapped[t] ? (need[t] - c->mapped[t]) / piece : 0);
        }
        const size_t n_fresh = first_new[n_tensors];
        if (n_fresh > 0) {
            // memory for every tensor first, then the mappings: a failure anywhere leaves the cache as it was
            const hipMemAllocationProp prop = device_memory_prop(c->cfg.device);
            std::vector<size_t> before(n_tensors);
            for (size_t t = 0; t < n_tensors; ++t) before[t] = c->chunks[t].size();
            std::vector<hipMemGenericAllocationHandle_t> fresh;
            fresh.reserve(n_fresh);
            for (size_t i = 0; i < n_fresh; ++i) {
                hipMemGenericAllocationHandle_t h;
                const hipError_t ce = hipMemCreate(&h, piece, &prop, 0);
                if (ce != hipSuccess) {
                    (void)hipGetLastError();
                    for (auto& f : fresh) (void)hipMemRelease(f);
                    // (out of memory reads as the reference's message; anything else keeps the runtime's own text)
                    throw StatusError(PA_NOT_ALLOCATED, ce == hipErrorOutOfMemory ? std::string(too_large)
                                                            : std::string("creating KV-cache memory failed: ") + hipGetErrorString(ce));
                }
                fresh.push_back(h);
            }
            hipMemAccessDesc access{};
            access.location = prop.location;
            access.flags = hipMemAccessFlagsProtReadWrite;
            for (size_t t = 0; t < n_tensors; ++t) {
                for (size_t i = first_new[t]; i < first_new[t + 1]; ++i) {
                    const size_t off = c->mapped[t] + (i - first_new[t]) * piece;
                    uint8_t* at = static_cast<uint8_t*>(c->tensor(t)) + off;
                    hipError_t e = hipMemMap(at, piece, 0, fresh[i], 0);
                    bool listed = false;
                    if (e == hipSuccess) {
                        c->chunks[t].push_back({fresh[i], off, piece});
                        listed = true;
                        e = hipMemSetAccess(at, piece, &access, 1);
                    }
                    if (e != hipSuccess) {
                        (void)hipGetLastError();
                        for (size_t u = listed ? i + 1 : i; u < n_fresh; ++u) (void)hipMemRelease(fresh[u]);
                        drop_chunks(c, before);
                        throw StatusError(PA_NOT_ALLOCATED, std::string("mapping KV-cache memory failed: ") + hipGetErrorString(e));
                    }
                }
            }
            // new blocks start as zeros (rows no token has been written to are then harmless in any format)
            // (a failure here also unmaps and releases what this call made: the next growth maps the same offsets)
            hipError_t ze = hipSuccess;
            for (size_t t = 0; t < n_tensors && ze == hipSuccess; ++t)
                if (need[t] > c->mapped[t])
                    ze = hipMemsetAsync(static_cast<uint8_t*>(c->tensor(t)) + c->mapped[t], 0, need[t] - c->mapped[t], s);
            if (ze == hipSuccess) ze = hipStreamSynchronize(s);
            if (ze != hipSuccess) {
                (void)hipGetLastError();
                (void)hipStreamSynchronize(s);
                drop_chunks(c, before);
                throw StatusError(PA_GENERAL_ERROR, std::string("clearing new KV-cache memory failed: ") + hipGetErrorString(ze));
            }
            for (size_t t = 0; t < n_tensors; ++t) c->mapped[t] = std::max(c->mapped[t], need[t]);
        }
        c->num_blocks = num_kv_blocks;
    });
}

int32_t pa_kv_cache_get(const pa_kv_cache* c, int32_t layer, void** key_cache, void** value_cache) {
    if (!c || !key_cache || !value_cache) return PA_INVALID_C_PARAM;
    if (layer < 0 || layer >= c->cfg.num_layers) return PA_OUT_OF_BOUNDS;
    *key_cache = c->key[layer];
    *value_cache = c->value[layer];
    return PA_OK;
}

int32_t pa_kv_cache_copy_blocks(pa_kv_cache* c, const int32_t* src, const int32_t* dst, int32_t count) {
    if (!c) return PA_INVALID_C_PARAM;
    return guarded(c, [&] {
        PA_REQUIRE(count >= 0 && (count == 0 || (src && dst)), PA_INVALID_C_PARAM, "src/dst missing");
        for (int32_t i = 0; i < count; ++i)
            PA_REQUIRE(src[i] >= 0 && dst[i] >= 0 && (uint64_t)src[i] < c->num_blocks && (uint64_t)dst[i] < c->num_blocks,
                       PA_OUT_OF_BOUNDS, "block index outside the cache");
        if (count == 0) return;
        HIP_CHECK(hipSetDevice(c->cfg.device));
        hipStream_t s = static_cast<hipStream_t>(c->cfg.stream);
        // The pairs of one launch are copied side by side, the reference copies them one after the other: a pair that
        // reads what an earlier pair writes, or writes what an earlier pair reads or writes, starts a new launch.
        std::vector<int32_t> list;
        list.reserve(2 * (size_t)count);
        std::vector<int32_t> cuts{0};  // first pair of every launch
        {
            std::vector<uint8_t> role(c->num_blocks, 0);  // 1 = read, 2 = written by the launch being formed
            std::vector<int32_t> touched;
            for (int32_t i = 0; i < count; ++i) {
                if (src[i] == dst[i]) continue;
                if (role[src[i]] == 2 || role[dst[i]] != 0) {
                    for (int32_t b : touched) role[b] = 0;
                    touched.clear();
                    cuts.push_back((int32_t)(list.size() / 2));
                }
                role[src[i]] = std::max<uint8_t>(role[src[i]], 1);
                role[dst[i]] = 2;
                touched.push_back(src[i]);
                touched.push_back(dst[i]);
                list.push_back(src[i]);
                list.push_back(dst[i]);
            }
        }
        if (list.empty()) return;
        cuts.push_back((int32_t)(list.size() / 2));
        HIP_CHECK(hipStreamSynchronize(s));  // an earlier call's launches may still read the list
        c->pairs.reserve(list.size() * sizeof(int32_t));
        HIP_CHECK(hipMemcpyAsync(c->pairs.p, list.data(), list.size() * sizeof(int32_t), hipMemcpyHostToDevice, s));
        for (size_t k = 0; k + 1 < cuts.size(); ++k)
            HIP_CHECK(pa::launch_copy_blocks(s, c->base_table.as<void*>(),
                                             c->base_table.as<uint64_t>() + c->chunks.size(), (int)c->chunks.size(),
                                             c->pairs.as<int32_t>() + 2 * cuts[k], cuts[k + 1] - cuts[k],
                                             *std::max_element(c->block_bytes.begin(), c->block_bytes.end())));
        HIP_CHECK(hipStreamSynchronize(s));  // `list` is pageable and leaves scope; the reference's copy is synchronous too
    });
}

int32_t pa_normalize_num_kv_blocks(uint64_t num_kv_blocks, uint64_t cache_size_gib, uint64_t block_size,
                                   uint64_t block_bytes_all_layers, uint64_t total_memory, uint64_t* out) {
    return guarded<NoObj>(nullptr, [&] {
        PA_REQUIRE(out, PA_INVALID_C_PARAM, "out is null");
        PA_REQUIRE(block_size > 0 && block_bytes_all_layers > 0, PA_PARAMETER_MISMATCH, "block sizes must be positive");
        uint64_t n = num_kv_blocks;
        if (cache_size_gib > 0 && n == 0) {
            const uint64_t budget = cache_size_gib << 30;
            PA_REQUIRE(budget <= total_memory, PA_GENERAL_ERROR,
                       "Requested cache size is larger than available memory size on the system.");
            // the largest token target whose blocks fit the budget, in whole blocks
            n = budget / block_bytes_all_layers;
        } else if (n > 0) {
            PA_REQUIRE(n <= total_memory / block_bytes_all_layers, PA_GENERAL_ERROR,
                       "Requested cache blocks require more memory than available on the system.");
        }
        *out = n;
    });
}

}  // extern "C"
