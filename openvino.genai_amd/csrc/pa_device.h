// Shared device-side helpers and kernel launch declarations of the gfx950 PagedAttention library.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace pa {

enum : int { DT_F16 = 0, DT_BF16 = 1, DT_U8 = 2, DT_U4 = 3 };

constexpr int WAVE = 64;

// bytes of one cached row of D elements: 16-bit values; `f32 scale | f32 zero-point | D codes` (u8); the same header
// and two codes per byte (u4)
__host__ __device__ inline int row_bytes(int D, int dt) { return dt == DT_U8 ? D + 8 : dt == DT_U4 ? D / 2 + 8 : D * 2; }
__host__ __device__ inline int ceil_div(int a, int b) { return (a + b - 1) / b; }

// ---- 16-bit float bit patterns <-> f32 (device) ----------------------------------------------
__device__ inline float half_bits_to_float(uint16_t h) {
    return (float)__builtin_bit_cast(_Float16, h);
}
__device__ inline uint16_t float_to_half_bits(float f) {  // round to nearest even
    return __builtin_bit_cast(uint16_t, (_Float16)f);
}
__device__ inline float bf16_bits_to_float(uint16_t b) {
    return __builtin_bit_cast(float, (uint32_t)b << 16);
}
__device__ inline uint16_t float_to_bf16_bits(float f) {  // round to nearest even, NaN kept quiet
    uint32_t x = __builtin_bit_cast(uint32_t, f);
    if ((x & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((x >> 16) | 0x40u);
    x += 0x7fffu + ((x >> 16) & 1u);
    return (uint16_t)(x >> 16);
}
template <int DT>
__device__ inline float load16(uint16_t v) {
    return DT == DT_F16 ? half_bits_to_float(v) : bf16_bits_to_float(v);
}
template <int DT>
__device__ inline uint16_t store16(float f) {
    return DT == DT_F16 ? float_to_half_bits(f) : float_to_bf16_bits(f);
}

// ---- wave-wide reductions (64 lanes) ----------------------------------------------------------
__device__ inline float wave_max(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, WAVE));
    return v;
}
__device__ inline float wave_min(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = fminf(v, __shfl_xor(v, o, WAVE));
    return v;
}
__device__ inline float wave_sum(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, WAVE);
    return v;
}

// ---- reductions over the 16 lanes of a row (a row of a DPP row: lanes 16 k .. 16 k + 15) ----------------------
// Four cross-lane steps each; every lane ends up with the result.
template <int CTRL>
__device__ __forceinline__ float dpp_f(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, false));
}
__device__ __forceinline__ float row16_min(float v) {
    v = fminf(v, dpp_f<0xB1>(v));   // quad_perm [1, 0, 3, 2]
    v = fminf(v, dpp_f<0x4E>(v));   // quad_perm [2, 3, 0, 1]
    v = fminf(v, dpp_f<0x141>(v));  // row_half_mirror: the other quad of the eight
    return fminf(v, dpp_f<0x140>(v));  // row_mirror: the other eight of the sixteen
}
__device__ __forceinline__ float row16_max(float v) {
    v = fmaxf(v, dpp_f<0xB1>(v));
    v = fmaxf(v, dpp_f<0x4E>(v));
    v = fmaxf(v, dpp_f<0x141>(v));
    return fmaxf(v, dpp_f<0x140>(v));
}
// ... and over the 8 lanes of a half row
__device__ __forceinline__ float row8_min(float v) {
    v = fminf(v, dpp_f<0xB1>(v));
    v = fminf(v, dpp_f<0x4E>(v));
    return fminf(v, dpp_f<0x141>(v));
}
__device__ __forceinline__ float row8_max(float v) {
    v = fmaxf(v, dpp_f<0xB1>(v));
    v = fmaxf(v, dpp_f<0x4E>(v));
    return fmaxf(v, dpp_f<0x141>(v));
}
__device__ __forceinline__ float row16_sum(float v) {
    v += dpp_f<0xB1>(v);
    v += dpp_f<0x4E>(v);
    v += dpp_f<0x141>(v);
    return v + dpp_f<0x140>(v);
}

// ---- one K or V row into a u8 cache row ---------------------------------------------------------
// A 64-lane wave quantises one row of D = 64 * EPL elements: `f32 scale | f32 zero-point | D codes` with
//   scale = (max - min) / 255  (a zero range takes 1e-4),  zp = -min / scale,
//   code  = clamp(rne(fma(x, 1/scale, zp)), 0, 255),
// every operation in IEEE binary32 (no contraction), so that the bytes are reproducible on any IEEE host.
// `raw` holds the lane's EPL consecutive elements (bit patterns of QDT), elements lane * EPL ..; `dst` is the row's
// first byte.  A row shorter than 64 * EPL elements: the surplus lanes hold copies of other lanes' elements (which
// leaves minimum and maximum alone), pass those lanes' numbers and `store` = false.
template <int QDT, int EPL>
__device__ __forceinline__ void quantize_row_u8(const uint16_t (&raw)[EPL], uint8_t* dst, const int lane, const bool store = true) {
#pragma clang fp contract(off)
    float x[EPL];
#pragma unroll
    for (int e = 0; e < EPL; ++e) x[e] = load16<QDT>(raw[e]);
    float mn = x[0], mx = x[0];
#pragma unroll
    for (int e = 1; e < EPL; ++e) { mn = fminf(mn, x[e]); mx = fmaxf(mx, x[e]); }
    mn = wave_min(mn);
    mx = wave_max(mx);
    float scale = (mx - mn) / 255.0f;
    if (scale == 0.0f) scale = 0.0001f;
    const float zp = -mn / scale;
    const float inv = 1.0f / scale;
    uint32_t packed = 0;
#pragma unroll
    for (int e = 0; e < EPL; ++e) {
        float v = rintf(__fmaf_rn(x[e], inv, zp));
        v = fminf(fmaxf(v, 0.0f), 255.0f);
        packed |= (uint32_t)(int)v << (8 * e);
    }
    if (!store) return;
    if (lane == 0) *reinterpret_cast<float2*>(dst) = make_float2(scale, zp);
    uint8_t* c = dst + 8 + lane * EPL;
    if constexpr (EPL == 4) *reinterpret_cast<uint32_t*>(c) = packed;
    else if constexpr (EPL == 2) *reinterpret_cast<uint16_t*>(c) = (uint16_t)packed;
    else *c = (uint8_t)packed;
}
// The lane's EPL consecutive elements of a row of 16-bit values.
template <int EPL>
__device__ __forceinline__ void load_row16(const uint16_t* src, uint16_t (&raw)[EPL]) {
    if constexpr (EPL == 4) {
        const uint2 v = *reinterpret_cast<const uint2*>(src);
        raw[0] = v.x & 0xffff; raw[1] = v.x >> 16; raw[2] = v.y & 0xffff; raw[3] = v.y >> 16;
    } else if constexpr (EPL == 2) {
        const uint32_t v = *reinterpret_cast<const uint32_t*>(src);
        raw[0] = v & 0xffff; raw[1] = v >> 16;
    } else {
        raw[0] = src[0];
    }
}

// ---- step metadata as the kernels see it (all device pointers) --------------------------------
struct StepDev {
    const int32_t* past_lens;             // [B]
    const int32_t* subsequence_begins;    // [B+1]
    const int32_t* block_indices_begins;  // [B+1]
    const int32_t* score_window;          // [B], already clamped to [0, q_len]
    const int32_t* score_offsets;         // [B+1] prefix sum of past+new
    const int32_t* token_seq;             // [T] sequence of each token
    const int32_t* gtiles;                // [n_gtiles] token tiles of the shape-generic attention kernel: up to eight
                                          // consecutive tokens of one sequence, first token * 8 + (count - 1)
    int32_t n_gtiles;
    int32_t B, T;
    int32_t sliding_window;
    float scale;
};

struct Shape {
    int32_t Hq, Hkv, D, bs;
};

// ---- launches (defined in the .hip files) ------------------------------------------------------
// New K/V rows into the paged caches (u8: per-row asymmetric quantisation).
hipError_t launch_kv_append(hipStream_t s, const StepDev& st, const Shape& sh, int q_dtype, int kv_dtype,
                            const void* key, const void* value, void* key_cache, void* value_cache,
                            const int32_t* block_indices);

// Copy-on-write: block pairs[2 i] -> pairs[2 i + 1] in each of the n_tensors tensors whose base addresses `bases`
// and block sizes `tensor_block_bytes` list (device arrays); one launch for all of them.
hipError_t launch_copy_blocks(hipStream_t s, void* const* bases, const uint64_t* tensor_block_bytes, int n_tensors,
                              const int32_t* pairs, int count, size_t max_block_bytes);

struct AttnWorkspace {
    float* part_acc;   // [T*Hq*nsplit, D] (D: the value head size)
    float* part_ml;    // [T*Hq*nsplit, 2]
    float* final_ml;   // [T*Hq, 2]
    float* logits;     // [Hq, total_scores] raw scaled logits of single-token sequences (scores only)
    int32_t nsplit;
    int32_t total_scores;
    const float* alibi = nullptr;  // [Hq] ALiBi slopes, or null: logit += slope * (key position - query position)
};

// What the shape-generic kernels take: a head size and an element type per cache tensor (query and key rows have Dk
// elements, value and output rows Dv; both multiples of 8, at most GENERIC_MAX_HEAD_SIZE).
constexpr int GENERIC_MAX_HEAD_SIZE = 512;
struct GenericShape {
    int32_t Hq, Hkv, Dk, Dv, bs, kdt, vdt;
};
// What one wave of the shape-generic attention kernel serves: `rows` (1, 2, 4 or 8) query rows that share every cache
// row it reads -- `heads` heads of one kv head's group (a power of two) for each of `tokens` consecutive tokens of one
// sequence -- as many as keep the wave's query rows within 8 KB of LDS.  Steps without multi-token sequences take one
// token per wave.
struct GenericPlan {
    int rows, heads, tokens;
};
inline GenericPlan generic_plan(const GenericShape& sh, bool multi_token) {
    const int G = sh.Hq / sh.Hkv;
    int most = 8;
    while (most > 1 && most * sh.Dk > 1024) most >>= 1;
    GenericPlan p;
    p.heads = 1;
    while (p.heads < most && p.heads < G) p.heads <<= 1;
    p.tokens = multi_token ? most / p.heads : 1;
    p.rows = p.heads * p.tokens;
    return p;
}
hipError_t launch_attention_generic(hipStream_t s, const StepDev& st, const GenericShape& sh, int q_dtype,
                                    const void* query, const void* key_cache, const void* value_cache,
                                    const int32_t* block_indices, const AttnWorkspace& ws, void* out, float* scores,
                                    int32_t max_kv_len, hipEvent_t ev0, hipEvent_t ev1);
hipError_t launch_kv_append_generic(hipStream_t s, const StepDev& st, const GenericShape& sh, int q_dtype, const void* key,
                                    const void* value, void* key_cache, void* value_cache, const int32_t* block_indices);

// What a workgroup of the u8 decode kernel needs to start fetching KV blocks, resolved on the host when the block
// table is set: one entry per (listed sequence, split), read with one scalar load instead of a chain of dependent
// loads through the step arrays and the table.
struct DecodeDesc {
    int32_t b, t;           // sequence and its token row
    int32_t kv_len, first;  // context length (new token included) and first visible position
    int32_t tb, te;         // KV blocks [tb, te) of this split
    int32_t table_off;      // first entry of the sequence's block table
    int32_t score_off;      // first entry of the sequence in `scores`
    int32_t last_id;        // physical id of the block that holds position kv_len - 1
    int32_t pad[7];
    int32_t ids[16];        // physical ids of the split's first 16 blocks (0 beyond te)
};
static_assert(sizeof(DecodeDesc) == 128, "one descriptor = 128 bytes");

// Arguments of the u8 decode kernel family (pa_decode_u8.hip).
struct DecodeArgs {
    StepDev st;
    Shape sh;
    const uint16_t* query;        // [T, Hq*D], T == B (one token per sequence)
    const uint8_t* key_cache;     // [num_blocks, Hkv, 32, D+8]
    const uint8_t* value_cache;
    const int32_t* block_indices;
    const int32_t* seq_list;      // sequences this launch covers (single-token ones); null = all B
    const DecodeDesc* descs;      // u8 kernel: [n_seqs][nsplit]
    const uint16_t* key;          // with fuse_append: the step's new K / V rows [T, Hkv*D], which the workgroup that
    const uint16_t* value;        // owns a sequence's last block writes (u8: quantises) into the caches itself
    int32_t fuse_append;
    int32_t n_seqs;
    int32_t G;                    // query heads per kv head (<= 16)
    int32_t nsplit;               // workgroups per (sequence, kv head)
    int32_t max_tiles;            // most KV blocks any workgroup walks
    int32_t want_scores;
    int32_t total_scores;
    int32_t waves;                // waves per workgroup
    int32_t table_off;            // byte offset of the block-table slice in LDS (set by the launcher)
    uint16_t* out;                // [T, Hq*D]
    float* part_acc;              // nsplit > 1: [T*Hq*nsplit, D] un-normalised
    float* part_ml;               // nsplit > 1: [T*Hq*nsplit, 2] (max in the log2 domain, denominator)
    float* final_ml;              // [T*Hq, 2]
    _Float16* group_scores;       // nsplit == 1: [Hkv, total_scores] per-kv-head score sums on their way to the score kernel
    _Float16* p_split;            // nsplit > 1: [Hq, p_split_stride(total_scores, B)] probabilities relative to the
                                  // split maximum; a sequence's run starts at p_split_offset (16-byte aligned)
};
// Layout of the per-head split probabilities: every sequence's run starts on a multiple of 8 elements.
__host__ __device__ inline long p_split_offset(long score_offset, int b) { return ((score_offset + 7) & ~7L) + 8L * b; }
__host__ __device__ inline long p_split_stride(long total_scores, int B) { return total_scores + 8L * B + 8; }

size_t decode_u8_lds_bytes(int D, int G, int max_tiles, bool want_scores, int waves, int32_t* table_off, int block_size);
// ev0 / ev1 (may be null) are recorded right before and after the main kernel.
hipError_t launch_decode_u8(hipStream_t s, const DecodeArgs& a, int q_dtype, float* scores, int max_kv_len,
                            hipEvent_t ev0, hipEvent_t ev1);

// ---- block-sparse prefill (XAttention) -----------------------------------------------------------
// Blocks and strided groups are counted by absolute position: query / key block I covers positions
// [I * xb, (I + 1) * xb), strided group i covers [i * S, (i + 1) * S); xb and S are powers of two, S <= 32 <= xb.
constexpr int XATT_KEY_TILE = 64;   // strided key groups one workgroup of the logits kernel covers (rows of logits are padded to 128)
struct XattSeq {            // one sequence of the step that runs block-sparse
    int32_t b;              // sequence
    int32_t qb0, nqb;       // first query block of the chunk and how many it touches
    int32_t nkb;            // key blocks = qb0 + nqb
    int32_t words;          // 32-bit words of one mask row: ceil(nkb / 32)
    int32_t qs0, nqs;       // first strided query group of the chunk and how many it touches
    int32_t nks;            // strided key groups: ceil(kv_len / S)
    int32_t ld;             // row length of the strided logits (nks rounded up to 128)
    float threshold;
    int64_t logit_off;      // strided logits [Hq][nqs rounded up to 32][ld] floats (log2 domain)
    int64_t sum_off;        // block sums [Hq][nqb][nkb] floats
    int64_t mask_off;       // retained key blocks, [Hq][nqb][words] words, bit J % 32 of word J / 32
};
struct XattDev {            // what the attention and score kernels need of it (all device pointers)
    const XattSeq* seqs;
    const int32_t* seq_of;  // [B]: index into seqs, -1 for a dense sequence
    const uint32_t* mask;
    const int32_t* item_tiles;  // per (sparse work item, kv head): how many of the item's KV blocks some row of it
                                // still needs, then their offsets from the item's first block, ascending
    int32_t tiles_stride;       // entries per (item, kv head): 1 + the longest item's block count
    int32_t xb_shift;           // log2(xb)
};

// The 16-bit-cache decode kernel (pa_decode16.hip): takes the arguments of the u8 family and leaves split partials,
// per-kv-head score sums and split probabilities in its layouts (table_off is set by the launcher).
// floats of the 16-bit decode kernel's per-(block, head) maxima in LDS (the probabilities behind them stay 16-byte aligned)
__host__ __device__ inline int decode16_snap_floats(int max_tiles, int G) { return (max_tiles * G + 3) & ~3; }
size_t decode16_lds_bytes(int D, int G, int max_tiles, bool want_scores);
size_t decode16_table_bytes(int max_tiles, int block_size);  // the block-table slice behind it
hipError_t launch_decode16(hipStream_t s, const DecodeArgs& a, int dtype, float* scores, int max_kv_len, hipEvent_t ev0,
                           hipEvent_t ev1);
// The merge and score kernels of the decode family on their own.
hipError_t preload_decode_u8();
hipError_t preload_decode16();
hipError_t launch_decode_merge(hipStream_t s, const DecodeArgs& a, int q_dtype);
hipError_t launch_decode_scores(hipStream_t s, const DecodeArgs& a, float* scores, int max_kv_len);
hipError_t launch_decode_post(hipStream_t s, const DecodeArgs& a, int q_dtype, float* scores, int max_kv_len);

// One work item of the 16-bit-cache MFMA kernel: a tile of query tokens against a range of KV blocks.
struct PrefillItem {
    int32_t b;        // sequence
    int32_t q0, nq;   // first query token of the tile (within the sequence) and how many
    int32_t tb, te;   // KV blocks [tb, te) of the sequence this item walks
    int32_t split;    // index of this range among the nsplit ranges of the tile
    int32_t nsplit;
    int32_t pad;
};

// Arguments of the 16-bit-cache MFMA kernel (pa_prefill16.hip).
struct PrefillArgs {
    StepDev st;
    Shape sh;
    const uint16_t* query;
    const uint8_t* key_cache;     // [num_blocks, Hkv, 32, D] f16 / bf16, or [.., D+8] u8 rows
    const uint8_t* value_cache;
    const int32_t* block_indices;
    const PrefillItem* items;
    const int32_t* tok_nsplit;    // [T] ranges the context of each token's tile was cut into
    const int32_t* merge_tokens;  // [n_merge] the tokens with more than one range, ascending
    int32_t n_merge;
    int32_t n_items;
    int32_t n_wide;               // the first n_wide items have more than 16 query rows, the others at most 16
    int32_t G;                    // query heads per kv head
    int32_t max_split;            // stride of the partial buffers
    uint16_t* out;
    float* final_ml;              // [T*Hq, 2] natural-log maximum and denominator per row
    float* part_acc;              // [T*Hq*max_split, D] un-normalised partial rows
    float* part_ml;               // [T*Hq*max_split, 2] (max in the log2 domain, denominator)
    int32_t n_sparse;             // the last n_sparse items belong to block-sparse sequences (see XattDev)
    XattDev xatt;
    // n_single items belong to single-token sequences (16-bit caches).  In a step without dense chunks they sit
    // together in front of the block-sparse items, and a call that hands those sequences to the decode kernel
    // (skip_single) passes their items and output rows over; next to dense chunks they may be listed between the
    // chunks' items, and skip_single is never set.
    int32_t n_single;
    const int32_t* single_idx;    // [B]: index among the single-token sequences, -1 for the others
    int32_t skip_single;
    // Scores of single-token sequences that are work items of this kernel (16-bit caches, next to dense chunks): the
    // kernel keeps every head's probabilities, relative to the running maximum at their 32-token tile, and that
    // maximum per (head, tile) in LDS while it walks an item, and leaves them here when the item is done;
    // `launch_single_scores` turns them into scores once the rows' final maxima and denominators are known.  Null:
    // nothing is left (the score replay serves those sequences).
    _Float16* p_out;              // [tiles][Hq][32]: a sequence's tiles start at tile_max_offset(score offset, b)
    float* tile_max;              // [tiles][Hq]
};
// What an item of a single-token sequence may keep in LDS: 64 G bytes of probabilities and 4 G of maxima per tile.
constexpr int SINGLE_STASH_BYTES = 20480;
__host__ __device__ inline int single_item_max_tiles(int G) { return SINGLE_STASH_BYTES / (68 * G); }
// Tiles of the sequences of a step, one after the other: a sequence of kv_len positions takes ceil(kv_len / 32).
__host__ __device__ inline long tile_max_offset(long score_offset, int b) { return (score_offset >> 5) + b; }
__host__ __device__ inline long tile_max_count(long total_scores, int B) { return (total_scores >> 5) + B + 1; }
// Scores of single-token sequences from the probabilities the matrix kernel left (after its merge kernel):
// score[pos] = sum over heads of p[h][pos] * 2^(tile maximum - final maximum) / denominator.  Runs as extra workgroups
// of the score replay's launch (rows of the grid behind the sequences', one per listed sequence; `gx` workgroups of
// 2048 positions each per row): both wait for the same merge, both are short and bound by latency.
struct SingleScores {
    const _Float16* p_out;   // null: no such rows
    const float* tile_max;
    const int32_t* seq_list;
    int32_t n_seqs, gx;
};
// The matrix kernel's rows whose context was cut into several ranges: what folding their partials takes.  The fold
// runs as a launch of its own or, when a score launch follows anyway, as extra workgroups of that launch (`n_wg` of
// them, 16 rows each); the score rows then form the maximum and denominator of such a row from the partial ones
// themselves instead of waiting for `final_ml`.  n_merge == 0: no such rows.
struct MergeRows {
    const float* part_acc;        // [T*Hq*max_split, D] un-normalised partial rows
    const float* part_ml;         // [T*Hq*max_split, 2] (max in the log2 domain, denominator)
    float* final_ml;              // [T*Hq, 2]
    uint16_t* out;
    const int32_t* merge_tokens;  // [n_merge]
    const int32_t* tok_nsplit;    // [T]
    const int32_t* single_idx;    // [B]
    const int32_t* token_seq;     // [T]
    int32_t n_merge, max_split, skip_single, Hq;
    int32_t n_wg;                 // workgroups of 256 threads that fold the rows: ceil(n_merge * Hq / 16)
};
inline MergeRows merge_rows_of(const PrefillArgs& a) {
    MergeRows m{};
    m.part_acc = a.part_acc;
    m.part_ml = a.part_ml;
    m.final_ml = a.final_ml;
    m.out = a.out;
    m.merge_tokens = a.merge_tokens;
    m.tok_nsplit = a.tok_nsplit;
    m.single_idx = a.single_idx;
    m.token_seq = a.st.token_seq;
    m.n_merge = a.n_merge;
    m.max_split = a.max_split;
    m.skip_single = a.skip_single;
    m.Hq = a.sh.Hq;
    m.n_wg = (int32_t)(((long)a.n_merge * a.sh.Hq + 15) / 16);
    return m;
}
#if defined(__HIPCC__)
// Natural-log maximum and denominator of query row `rid` (token `tok`): from `final_ml`, or folded from the row's
// partial ones when its context was cut into ranges that `m` describes.  (The fold is a call, not inline code: inside
// the replay's row loop it would cost the kernel 16 registers.)
__device__ inline __attribute__((noinline)) float2 fold_max_and_sum(const float2* pm, int ns) {
    constexpr float LN2_ = 0.6931471805599453f;
    float M = -INFINITY;
    for (int s = 0; s < ns; ++s) M = fmaxf(M, pm[s].x);
    float L = 0.0f;
    for (int s = 0; s < ns; ++s) {
        const float2 v = pm[s];
        L += v.x == -INFINITY ? 0.0f : v.y * __builtin_amdgcn_exp2f(v.x - M);
    }
    return make_float2(M * LN2_, L);
}
// The same fold as inline code with four partial pairs in flight at a time (running maximum and rescaled sum), for
// places with registers to spare: a round trip per four ranges instead of one per range.
__device__ __forceinline__ float2 fold_max_and_sum_wide(const float2* pm, int ns) {
    constexpr float LN2_ = 0.6931471805599453f;
    float M = -INFINITY, L = 0.0f;
    for (int s0 = 0; s0 < ns; s0 += 4) {
        float2 v[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) v[j] = pm[min(s0 + j, ns - 1)];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            if (s0 + j >= ns || v[j].x == -INFINITY) continue;
            const float Mn = fmaxf(M, v[j].x);
            L = L * __builtin_amdgcn_exp2f(M - Mn) + v[j].y * __builtin_amdgcn_exp2f(v[j].x - Mn);
            M = Mn;
        }
    }
    return make_float2(M * LN2_, L);
}
__device__ __forceinline__ float2 row_max_and_sum_wide(const float* __restrict__ final_ml, const MergeRows& m, int tok,
                                                       long rid) {
    const int ns = m.n_merge > 0 ? m.tok_nsplit[tok] : 1;
    if (ns <= 1) return *reinterpret_cast<const float2*>(final_ml + 2 * rid);
    return fold_max_and_sum_wide(reinterpret_cast<const float2*>(m.part_ml) + rid * m.max_split, ns);
}
__device__ __forceinline__ float2 row_max_and_sum(const float* __restrict__ final_ml, const MergeRows& m, int tok,
                                                  long rid) {
    const int ns = m.n_merge > 0 ? m.tok_nsplit[tok] : 1;
    if (ns <= 1) return *reinterpret_cast<const float2*>(final_ml + 2 * rid);
    return fold_max_and_sum(reinterpret_cast<const float2*>(m.part_ml) + rid * m.max_split, ns);
}

// Sixteen lanes per row, D / 16 channels each (16-byte loads; 8-byte ones when D / 16 is not a multiple of 4), four rows per wave, workgroup `wg` of 256 threads;
// ranges are folded in ascending order.  DT: type of the output rows.
template <int D, int DT>
__device__ __forceinline__ void merge_rows(const MergeRows& a, long wg) {
    typedef float f4_ __attribute__((ext_vector_type(4)));
    typedef uint32_t u4_ __attribute__((ext_vector_type(4)));
    constexpr float LN2_ = 0.6931471805599453f;
    constexpr int EPL = D / 16;
    const int l16 = threadIdx.x & 15;
    long idx = (wg * 256 + threadIdx.x) >> 4;
    const long n_rows = (long)a.n_merge * a.Hq;
    const bool live = idx < n_rows;
    idx = min(idx, n_rows - 1);  // (surplus groups repeat the last row and store nothing: no divergence around the shuffles)
    const int tok = a.merge_tokens[idx / a.Hq];
    const long row = (long)tok * a.Hq + idx % a.Hq;
    const bool mine = live && !(a.skip_single && a.single_idx[a.token_seq[tok]] >= 0);  // (else another kernel's row)
    const int ns = a.tok_nsplit[tok];
    float acc[EPL];
#pragma unroll
    for (int e = 0; e < EPL; ++e) acc[e] = 0.0f;
    float M, L;
    if (ns <= 16) {
        // lane s of the group holds range s: one round of loads instead of a dependent chain
        const float2 ml = l16 < ns ? *reinterpret_cast<const float2*>(a.part_ml + 2 * (row * a.max_split + l16))
                                   : make_float2(-INFINITY, 0.0f);
        M = ml.x;
#pragma unroll
        for (int o = 8; o > 0; o >>= 1) M = fmaxf(M, __shfl_xor(M, o, 16));
        const float f_mine = ml.x == -INFINITY ? 0.0f : __builtin_amdgcn_exp2f(ml.x - M);
        L = ml.y * f_mine;
#pragma unroll
        for (int o = 8; o > 0; o >>= 1) L += __shfl_xor(L, o, 16);
        // four ranges per round, loaded unconditionally (indices clamped, surplus ones weighted zero) so that
        // a round's loads are in flight together
        for (int s0 = 0; s0 < ns; s0 += 4) {
            float f[4];
            float v[4][EPL];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const long slot = row * a.max_split + min(s0 + j, ns - 1);
                f[j] = __shfl(f_mine, min(s0 + j, ns - 1), 16);
                if (s0 + j >= ns) f[j] = 0.0f;
                const float* pa = a.part_acc + slot * D + l16 * EPL;
                if constexpr (EPL % 4 == 0) {
#pragma unroll
                    for (int e = 0; e < EPL / 4; ++e) {
                        const f4_ x = reinterpret_cast<const f4_*>(pa)[e];
                        v[j][4 * e] = x[0], v[j][4 * e + 1] = x[1], v[j][4 * e + 2] = x[2], v[j][4 * e + 3] = x[3];
                    }
                } else {  // (a lane's channels start on an 8-byte boundary only)
#pragma unroll
                    for (int e = 0; e < EPL / 2; ++e) {
                        const float2 x = reinterpret_cast<const float2*>(pa)[e];
                        v[j][2 * e] = x.x, v[j][2 * e + 1] = x.y;
                    }
                }
            }
#pragma unroll
            for (int j = 0; j < 4; ++j)
#pragma unroll
                for (int e = 0; e < EPL; ++e)
                    acc[e] = fmaf(f[j] == 0.0f ? 0.0f : v[j][e], f[j], acc[e]);  // fully masked ranges hold nothing
        }
    } else {
        M = -INFINITY;
        for (int s = 0; s < ns; ++s) M = fmaxf(M, a.part_ml[2 * (row * a.max_split + s)]);
        L = 0.0f;
        for (int s = 0; s < ns; ++s) {
            const long slot = row * a.max_split + s;
            const float ms = a.part_ml[2 * slot];
            if (ms == -INFINITY) continue;
            const float f = __builtin_amdgcn_exp2f(ms - M);
            L += a.part_ml[2 * slot + 1] * f;
#pragma unroll
            for (int e = 0; e < EPL; ++e) acc[e] += a.part_acc[slot * D + l16 * EPL + e] * f;
        }
    }
    if (!mine) return;
    const float inv = L > 0.0f ? 1.0f / L : 0.0f;
    uint32_t o[EPL / 2];
#pragma unroll
    for (int e = 0; e < EPL / 2; ++e)
        o[e] = (uint32_t)store16<DT>(acc[2 * e] * inv) | ((uint32_t)store16<DT>(acc[2 * e + 1] * inv) << 16);
    uint16_t* dst = a.out + row * D + l16 * EPL;
    if constexpr (EPL == 8) *reinterpret_cast<u4_*>(dst) = u4_{o[0], o[1], o[2], o[3]};
    else if constexpr (EPL == 4) *reinterpret_cast<uint2*>(dst) = make_uint2(o[0], o[1]);
    else {
#pragma unroll
        for (int e = 0; e < EPL / 2; ++e) reinterpret_cast<uint32_t*>(dst)[e] = o[e];
    }
    if (l16 == 0) {
        a.final_ml[2 * row] = M * LN2_;
        a.final_ml[2 * row + 1] = L;
    }
}

__device__ __forceinline__ void single_scores_rows(const StepDev& st, const Shape& sh, const SingleScores& ss,
                                                   const float* __restrict__ final_ml, const MergeRows& mg,
                                                   float* __restrict__ scores, const int row, const int bx) {
    __shared__ float s_ml[2 * 256];  // [Hq][2]: final maximum (log2 domain), 1 / denominator
    constexpr float LOG2E_ = 1.4426950408889634f;
    if (bx >= ss.gx) return;
    const int b = ss.seq_list[row];
    const int t = st.subsequence_begins[b];
    const int kv_len = st.past_lens[b] + 1;
    const int first = st.sliding_window > 0 ? max(0, kv_len - st.sliding_window) : 0;
    const int W = st.score_window[b];
    const long so = st.score_offsets[b];
    float* out = scores + so;
    const int Hq = sh.Hq;
    for (int h = threadIdx.x; h < Hq; h += 256) {
        const float2 ml = row_max_and_sum_wide(final_ml, mg, t, (long)t * Hq + h);
        s_ml[2 * h] = ml.x * LOG2E_;
        s_ml[2 * h + 1] = ml.y > 0.0f ? 1.0f / ml.y : 0.0f;
    }
    __syncthreads();
    const long tg0 = tile_max_offset(so, b) * (long)Hq;  // [tile][head] of the sequence's first tile
    const _Float16* p = ss.p_out + tg0 * 32;
    const float* tmax = ss.tile_max + tg0;
    typedef _Float16 h8 __attribute__((ext_vector_type(8)));
    for (int pos = (bx * 256 + threadIdx.x) * 8; pos < kv_len; pos += ss.gx * 2048) {
        float s[8] = {0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f};
        if (W > 0 && pos + 7 >= first) {  // (tiles in front of the window's were not walked)
            const long th0 = (long)(pos >> 5) * Hq;
            constexpr int HU = 8;  // heads whose loads are in flight together
            for (int h0 = 0; h0 < Hq; h0 += HU) {  // heads in ascending order (fixed order, no atomics)
                h8 v[HU];
                float f[HU];
#pragma unroll
                for (int i = 0; i < HU; ++i) {
                    const int h = min(h0 + i, Hq - 1);
                    v[i] = *reinterpret_cast<const h8*>(p + (th0 + h) * 32 + (pos & 31));
                    f[i] = tmax[th0 + h];
                }
#pragma unroll
                for (int i = 0; i < HU; ++i) {
                    const int h = min(h0 + i, Hq - 1);
                    const float fac = h0 + i < Hq ? __builtin_amdgcn_exp2f(f[i] - s_ml[2 * h]) * s_ml[2 * h + 1] : 0.0f;
#pragma unroll
                    for (int e = 0; e < 8; ++e) s[e] += (float)v[i][e] * fac;
                }
            }
        }
#pragma unroll
        for (int e = 0; e < 8; ++e)
            if (pos + e < kv_len) out[pos + e] = pos + e >= first ? s[e] : 0.0f;
    }
}
#endif
// merge_later: the fold of the rows cut into ranges is left to the caller (`launch_scores_replay` takes it along).
hipError_t launch_prefill16(hipStream_t s, const PrefillArgs& a, int q_dtype, int kv_dtype, hipEvent_t ev0,
                            hipEvent_t ev1, bool merge_later = false);

// ---- block-sparse prefill (XAttention): the estimate's launch ---------------------------------
struct XattTile {           // one workgroup-sized piece of the strided logits: 32 query groups x 128 key groups
    int32_t x;              // index into the XattSeq list
    int32_t it, jc;         // query groups [32 it, 32 it + 32) of the chunk, key groups [128 jc, 128 jc + 128)
    int32_t pad;
};
struct XattArgs {
    StepDev st;
    Shape sh;
    const uint16_t* query;
    const uint8_t* key_cache;
    const int32_t* block_indices;
    const XattSeq* seqs;
    const int32_t* seq_of;      // [B]: index into seqs, -1 for a dense sequence
    const XattTile* tiles;
    int32_t nseq, ntiles;
    int32_t max_nqs, max_nqb, max_nkb;
    int32_t xb_shift, s_shift;  // log2 of the block size and of the stride
    float* logits;
    float* sums;
    uint32_t* mask;
    // the sparse work items of the matrix kernel (for the list of KV blocks each one needs)
    const PrefillItem* items;
    int32_t n_items;
    int32_t* item_tiles;
    int32_t tiles_stride;
    int32_t G;
};
// Estimate, block sums, selection and the work items' block lists, in stream order.
hipError_t launch_xattention(hipStream_t s, const XattArgs& a, int q_dtype, int kv_dtype);

// In-place re-rotation of the K rows of the listed physical blocks (device arrays; deltas are trig-table rows).
hipError_t launch_rotate(hipStream_t s, void* key_cache, int kv_dtype, const Shape& sh,
                         const int32_t* rotated_block_indices, const int32_t* deltas, int32_t deltas_per_block,
                         int32_t n_rotated, const float* trig_lut);

// Scores by replaying the last W query rows of every sequence against the positions they see (needs final_ml, or
// the partial maxima and denominators `mg` names for the rows cut into ranges; those rows' fold then runs as the last
// workgroups of the same launch).
hipError_t launch_scores_replay(hipStream_t s, const StepDev& st, const Shape& sh, int q_dtype, int kv_dtype,
                                const void* query, const void* key_cache, const int32_t* block_indices,
                                float* final_ml, float* scores, int32_t max_kv_len, const int32_t* seq_list,
                                int32_t n_seqs, const XattDev& xd, const SingleScores& ss, const MergeRows& mg);

// Block diversity of the evictable area (pa_rkv_diversity.hip).
struct RkvDivSeq {          // one sequence whose diversity is computed
    int32_t table_off;      // first entry of the sequence's block table
    int32_t first_block;    // logical block the evictable area starts at
    int32_t ev;             // evictable tokens, a multiple of the block size
    int32_t tok_off;        // first entry of the sequence in the per-token arrays (per head: + h * total_tok)
    int64_t out_off;        // first output value: [ev / block size, ev] floats
};
struct RkvDivArgs {
    const uint8_t* key_cache;
    const int32_t* block_indices;
    const RkvDivSeq* seqs;
    float4* stats;          // [Hkv, total_tok] workspace
    float* mean;            // [Hkv, total_tok] workspace: row mean of the similarities over the row's factor
    float* colsum;          // [nseq, Hkv, 1 + chunks_max, D] workspace: the total, then the chunks' sums
    float* out;
    int32_t Hkv;
    int32_t total_tok;
    int32_t chunks_max;     // rkv_diversity_chunks(longest area)
};
int rkv_diversity_chunks(int ev_max);
hipError_t launch_rkv_diversity(hipStream_t s, const RkvDivArgs& a, int kv_dtype, int D, int bs, int nseq, int ev_max);
// The same output for any head size that is a multiple of 8, any block size and u4 rows too, on
// the vector unit (pa_generic.hip); the column sums are kept per chunk of 256 tokens, as rkv_diversity_chunks counts.
hipError_t launch_rkv_diversity_generic(hipStream_t s, const RkvDivArgs& a, int kv_dtype, int D, int bs, int nseq, int ev_max);

}  // namespace pa
