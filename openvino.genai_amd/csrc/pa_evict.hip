// Score accumulation and block eviction with the state resident in HBM.
//
// Per tracked sequence (slot) and decoder layer the library keeps `double scores[cap]` and
// `uint64 counters[cap]`.  Three kernels:
//   evict_register_kernel : forward max-pool of the op's f32 scores + accumulate (+ lifetime counters)
//   evict_select_compact_kernel : one workgroup per (sequence, layer), everything an eviction of the plain
//                           modes needs in one launch: per-token score / counter staged through LDS (coalesced
//                           reads), per-block importance summed in token order, rank selection of the k lowest
//                           with ties to the lower index, the ascending list of evicted blocks, and the removal
//                           of their entries in place
//   evict_block_score / evict_rank / evict_list / evict_compact : the same steps as separate kernels, for the
//                           modes whose choice among blocks runs on the host in between (ADAPTIVE_RKV, KVCrush)
//                           and for areas too long for LDS
//   evict_rkv_push / evict_rkv_mean_pool : ADAPTIVE_RKV tracker -- the last `window` score vectors are kept
//                           in a ring per (slot, layer); the tracked score is their mean, max-pooled
//   evict_filtered_diversity_kernel : per block row of a registered diversity matrix, the mean over the
//                           columns of the blocks in the diversity set
// The choice among blocks that ADAPTIVE_RKV and KVCrush make at eviction time runs on the host (pa_select.h)
// on the block scores copied back: a few hundred values per (sequence, layer).
// All arithmetic is IEEE binary64 / integer in a fixed order, so results match a scalar CPU
// evaluation bit for bit.  HBM-bound: every tracked entry is read and written once per call.
#include <algorithm>
#include <atomic>
#include <cmath>
#include <cstring>
#include <exception>
#include <set>
#include <stdexcept>
#include <string>
#include <thread>
#include <vector>

#include "../../include/pa_amd.h"
#include "pa_device.h"
#include "host_parallel.h"
#include "pa_select.h"

namespace {

thread_local std::string g_evict_error;

struct StatusError : std::runtime_error {
    int32_t code;
    StatusError(int32_t c, const std::string& m) : std::runtime_error(m), code(c) {}
};
#define PA_REQUIRE(cond, code, msg)                    \
    do {                                               \
        if (!(cond)) throw StatusError((code), (msg)); \
    } while (0)
#define HIP_CHECK(expr)                                                                        \
    do {                                                                                       \
        hipError_t e_ = (expr);                                                                \
        if (e_ != hipSuccess)                                                                  \
            throw StatusError(e_ == hipErrorOutOfMemory ? PA_NOT_ALLOCATED : PA_GENERAL_ERROR, \
                              std::string(#expr) + ": " + hipGetErrorString(e_));              \
    } while (0)

enum : int32_t { RULE_SKIP = 0, RULE_INIT = 1, RULE_INIT_SNAPKV = 2, RULE_ADD = 3, RULE_ADD_SNAPKV = 4 };

struct RegEntry {       // one (sequence, layer) of a register call
    int64_t src_off;    // first tracked score inside scores.<layer>
    int64_t state_off;  // first entry of this (slot, layer) in the state arrays
    int32_t old_len;
    int32_t new_len;
    int32_t rule;
    int32_t snap;       // num_snapkv_scores (RULE_INIT_SNAPKV) or registered SnapKV scores (RULE_ADD_SNAPKV)
};

struct SelEntry {       // one (sequence, layer) of an evict / remove call
    int64_t state_off;
    int64_t list_off;   // first entry in the evicted-block list / block-score scratch
    int32_t len;        // tracked tokens
    int32_t n_blocks;   // evictable blocks (from tracked block 0)
    int32_t k;          // blocks to evict
    int32_t out_off;    // first entry of this pair's evicted blocks in the packed output (prefix sum of k)
};

__global__ __launch_bounds__(256) void evict_register_kernel(const RegEntry* __restrict__ entries,
                                                             const float* const* __restrict__ layer_scores,
                                                             double* __restrict__ scores,
                                                             unsigned long long* __restrict__ counters, int32_t layers,
                                                             int32_t pool, int32_t norm_sum) {
#pragma clang fp contract(off)
    const int l = blockIdx.z;
    const RegEntry e = entries[(long)blockIdx.y * layers + l];
    if (e.rule == RULE_SKIP) return;
    const float* src = layer_scores[l] + e.src_off;
    const int m = e.new_len;
    for (int i = blockIdx.x * 256 + threadIdx.x; i < m; i += gridDim.x * 256) {
        const int eff = min(pool, m - i);
        float best = src[i];
        for (int k = 1; k < eff; ++k) best = fmaxf(src[i + k], best);
        const double pv = (double)best;
        const long o = e.state_off + i;
        if (e.rule == RULE_INIT || e.rule == RULE_INIT_SNAPKV) {
            scores[o] = pv;
            if (norm_sum)
                counters[o] = (e.rule == RULE_INIT || i >= m - e.snap) ? (unsigned long long)(m - i)
                                                                       : (unsigned long long)e.snap;
        } else {
            const double old = i < e.old_len ? scores[o] : 0.0;
            scores[o] = old + pv;
            if (norm_sum) {
                if (e.rule == RULE_ADD)
                    counters[o] = i < e.old_len ? counters[o] + (unsigned long long)(m - e.old_len)
                                                : (unsigned long long)(m - i);
                else
                    counters[o] = i >= m - e.snap ? (unsigned long long)(m - i) : (unsigned long long)e.snap;
            }
        }
    }
}

// One workgroup per entry: importance of every evictable block, summed in token order.
__global__ __launch_bounds__(256) void evict_block_score_kernel(const SelEntry* __restrict__ entries,
                                                                const double* __restrict__ scores,
                                                                const unsigned long long* __restrict__ counters,
                                                                double* __restrict__ block_score, int32_t bsz,
                                                                int32_t norm_sum) {
#pragma clang fp contract(off)
    const SelEntry e = entries[blockIdx.x];
    double* bscore = block_score + e.list_off;
    for (int i = threadIdx.x; i < e.n_blocks; i += 256) {
        double acc = 0.0;
        for (int j = 0; j < bsz; ++j) {
            const long t = e.state_off + (long)i * bsz + j;
            acc += norm_sum ? scores[t] / (double)counters[t] : scores[t];
        }
        bscore[i] = acc != acc ? INFINITY : acc;  // a block whose score is not a number is never preferred
    }
}

// Rank of a block = number of blocks ordered before it (lower score, or equal score and lower
// index); the k lowest ranks are evicted.
__global__ __launch_bounds__(256) void evict_rank_kernel(const SelEntry* __restrict__ entries,
                                                         const double* __restrict__ block_score,
                                                         int32_t* __restrict__ flags) {
    const SelEntry e = entries[blockIdx.x];
    if (e.n_blocks <= 0 || e.k <= 0) return;
    const double* bscore = block_score + e.list_off;
    for (int i = threadIdx.x; i < e.n_blocks; i += 256) {
        const double si = bscore[i];
        int rank = 0;
        for (int j = 0; j < e.n_blocks; ++j) {
            const double sj = bscore[j];
            rank += (sj < si || (sj == si && j < i)) ? 1 : 0;
        }
        flags[e.list_off + i] = rank < e.k ? 1 : 0;
    }
}

__global__ __launch_bounds__(256) void evict_list_kernel(const SelEntry* __restrict__ entries,
                                                         const int32_t* __restrict__ flags,
                                                         int32_t* __restrict__ evicted) {
    const SelEntry e = entries[blockIdx.x];
    if (e.n_blocks <= 0 || e.k <= 0) return;
    const int32_t* f = flags + e.list_off;
    for (int i = threadIdx.x; i < e.n_blocks; i += 256) {
        if (!f[i]) continue;
        int pos = 0;
        for (int j = 0; j < i; ++j) pos += f[j];
        evicted[e.list_off + pos] = i;
    }
}

// In-place removal of the evicted blocks' entries: chunks are read whole before any of their
// elements is written, and an element only ever moves towards lower indices.
__global__ __launch_bounds__(256) void evict_compact_kernel(const SelEntry* __restrict__ entries,
                                                            const int32_t* __restrict__ evicted,
                                                            double* __restrict__ scores,
                                                            unsigned long long* __restrict__ counters, int32_t bsz,
                                                            int32_t norm_sum) {
    const SelEntry e = entries[blockIdx.x];
    if (e.k <= 0) return;
    const int32_t* list = evicted + e.list_off;
    constexpr int PER = 4;
    for (int base = 0; base < e.len; base += 256 * PER) {
        double sv[PER];
        unsigned long long cv[PER];
        int dst[PER];
#pragma unroll
        for (int r = 0; r < PER; ++r) {
            const int t = base + r * 256 + threadIdx.x;
            dst[r] = -1;
            if (t < e.len) {
                const int blk = t / bsz;
                int lo = 0, hi = e.k;  // first list entry >= blk
                while (lo < hi) {
                    const int mid = (lo + hi) >> 1;
                    if (list[mid] < blk) lo = mid + 1; else hi = mid;
                }
                const bool gone = lo < e.k && list[lo] == blk;
                if (!gone) {
                    dst[r] = t - lo * bsz;
                    sv[r] = scores[e.state_off + t];
                    if (norm_sum) cv[r] = counters[e.state_off + t];
                }
            }
        }
        __syncthreads();
#pragma unroll
        for (int r = 0; r < PER; ++r) {
            if (dst[r] >= 0) {
                scores[e.state_off + dst[r]] = sv[r];
                if (norm_sum) counters[e.state_off + dst[r]] = cv[r];
            }
        }
        __syncthreads();
    }
}

// Bytes of LDS the fused kernel needs for an entry: quotients [n_blocks][bsz + 1] doubles (the odd row length
// keeps the per-block sums free of bank conflicts), block scores, flags, the evicted list.
inline size_t select_lds_bytes(int64_t n_blocks, int64_t bsz, int64_t k) {
    return (size_t)(n_blocks * (bsz + 1) * 8 + n_blocks * 8 + n_blocks * 4 + ((k + 1) & ~1LL) * 4);
}

// One workgroup per entry: block scores, selection, list and compaction.  `lds_blocks` is the largest n_blocks of
// the launch (it fixes the carve-up); entries with k == 0 return at once.
__global__ __launch_bounds__(256) void evict_select_compact_kernel(const SelEntry* __restrict__ entries,
                                                                   double* __restrict__ scores,
                                                                   unsigned long long* __restrict__ counters,
                                                                   int32_t* __restrict__ out_list, int32_t bsz,
                                                                   int32_t norm_sum, int32_t lds_blocks) {
#pragma clang fp contract(off)
    extern __shared__ __align__(16) uint8_t sel_smem[];
    const SelEntry e = entries[blockIdx.x];
    if (e.k <= 0 || e.n_blocks <= 0) return;
    double* q = reinterpret_cast<double*>(sel_smem);                // [n_blocks][bsz + 1]
    double* bscore = q + (size_t)lds_blocks * (bsz + 1);            // [n_blocks]
    int32_t* flag = reinterpret_cast<int32_t*>(bscore + lds_blocks);  // [n_blocks]
    int32_t* list = flag + lds_blocks;                              // [k]
    const int tid = threadIdx.x;
    const int n_tok = e.n_blocks * bsz;
    for (int i = tid; i < n_tok; i += 256) {
        const long t = e.state_off + i;
        q[(i / bsz) * (bsz + 1) + i % bsz] = norm_sum ? scores[t] / (double)counters[t] : scores[t];
    }
    __syncthreads();
    for (int i = tid; i < e.n_blocks; i += 256) {
        double acc = 0.0;
        for (int j = 0; j < bsz; ++j) acc += q[i * (bsz + 1) + j];
        bscore[i] = acc != acc ? INFINITY : acc;  // a block whose score is not a number is never preferred
    }
    __syncthreads();
    for (int i = tid; i < e.n_blocks; i += 256) {
        const double si = bscore[i];
        int rank = 0;
        for (int j = 0; j < e.n_blocks; ++j) {
            const double sj = bscore[j];
            rank += (sj < si || (sj == si && j < i)) ? 1 : 0;
        }
        flag[i] = rank < e.k ? 1 : 0;
    }
    __syncthreads();
    for (int i = tid; i < e.n_blocks; i += 256) {
        if (!flag[i]) continue;
        int pos = 0;
        for (int j = 0; j < i; ++j) pos += flag[j];
        list[pos] = i;
        out_list[e.out_off + pos] = i;
    }
    __syncthreads();
    // removal in place: chunks are read whole before any of their elements is written, and an element only ever
    // moves towards lower indices
    constexpr int PER = 4;
    for (int base = 0; base < e.len; base += 256 * PER) {
        double sv[PER];
        unsigned long long cv[PER];
        int dst[PER];
#pragma unroll
        for (int r = 0; r < PER; ++r) {
            const int t = base + r * 256 + tid;
            dst[r] = -1;
            if (t < e.len) {
                const int blk = t / bsz;
                int lo = 0, hi = e.k;  // first list entry >= blk
                while (lo < hi) {
                    const int mid = (lo + hi) >> 1;
                    if (list[mid] < blk) lo = mid + 1; else hi = mid;
                }
                const bool gone = lo < e.k && list[lo] == blk;
                if (!gone) {
                    dst[r] = t - lo * bsz;
                    sv[r] = scores[e.state_off + t];
                    if (norm_sum) cv[r] = counters[e.state_off + t];
                }
            }
        }
        __syncthreads();
#pragma unroll
        for (int r = 0; r < PER; ++r) {
            if (dst[r] >= 0 && dst[r] != base + r * 256 + tid) {
                scores[e.state_off + dst[r]] = sv[r];
                if (norm_sum) counters[e.state_off + dst[r]] = cv[r];
            }
        }
        __syncthreads();
    }
}

// Token scores of the listed entries' evictable areas, packed one after the other (for the host's KVCrush step).
struct GatherEntry {
    int64_t state_off, dst_off;
    int32_t n;
    int32_t pad;
};
__global__ __launch_bounds__(256) void evict_gather_kernel(const GatherEntry* __restrict__ entries,
                                                           const double* __restrict__ scores, double* __restrict__ out) {
    const GatherEntry e = entries[blockIdx.x];
    for (int i = blockIdx.y * 256 + threadIdx.x; i < e.n; i += gridDim.y * 256) out[e.dst_off + i] = scores[e.state_off + i];
}

// Copies of float vectors between device buffers, all of a call in one launch (blockIdx.x = vector, .y = its part).
struct CopyEntry {
    const float* src;
    float* dst;
    int64_t n;
};
__global__ __launch_bounds__(256) void evict_copy_kernel(const CopyEntry* __restrict__ entries) {
    const CopyEntry e = entries[blockIdx.x];
    const int64_t step = (int64_t)gridDim.y * 256, first = (int64_t)blockIdx.y * 256 + threadIdx.x;
    if ((((uintptr_t)e.src | (uintptr_t)e.dst) & 15) == 0) {
        const float4* s4 = reinterpret_cast<const float4*>(e.src);
        float4* d4 = reinterpret_cast<float4*>(e.dst);
        const int64_t n4 = e.n / 4;
        for (int64_t i = first; i < n4; i += step) d4[i] = s4[i];
        for (int64_t i = n4 * 4 + first; i < e.n; i += step) e.dst[i] = e.src[i];
    } else {
        for (int64_t i = first; i < e.n; i += step) e.dst[i] = e.src[i];
    }
}

// KVCrush on the device (kvcrush.cpp:14-111), one workgroup per (sequence, layer) whose chosen blocks are thinned:
// the indicator bit of every token of the evictable area (1 for the half with the larger scores), the anchor point,
// and per block the Hamming distance between its bits and the anchor -- everything that walks tokens.  The host is
// left with one distance per block for the choice of the representatives (kvcrush.cpp:113-148, a std::sort whose
// order among equal distances is part of the contract).
// The reference picks the top half with std::partial_sort, so among tokens whose score equals the half's smallest one
// the choice is the library's: when not all of them fall on one side, `flags` says so and the host works that entry
// through from the scores themselves.
struct CrushEntry {
    int64_t state_off;   // first tracked score of this (slot, layer)
    int32_t n_tok;       // tokens of the evictable area
    int32_t dist_off;    // first entry of the block distances in the packed output
    int32_t anchor_off;  // first byte of this entry's anchor point (modes whose anchor the host supplies)
    int32_t pad;
};
__device__ __forceinline__ uint64_t score_key(double v) {  // ascending as unsigned integers; -0.0 and +0.0 alike
    uint64_t u = (uint64_t)__double_as_longlong(v);
    if (u == 0x8000000000000000ull) u = 0;
    return (u >> 63) ? ~u : (u | 0x8000000000000000ull);
}
__global__ __launch_bounds__(256) void evict_crush_kernel(const CrushEntry* __restrict__ entries,
                                                          const double* __restrict__ scores,
                                                          const uint8_t* __restrict__ host_anchors, int32_t* __restrict__ dist,
                                                          int32_t* __restrict__ flags, int32_t bsz, int32_t anchor_mode) {
    __shared__ uint32_t hist[256];
    __shared__ uint64_t s_prefix;
    __shared__ uint32_t s_rank, s_gt, s_eq;
    extern __shared__ uint32_t ones[];  // [bsz] indicator bits set per in-block position, then the anchor point
    const CrushEntry e = entries[blockIdx.x];
    const int tid = threadIdx.x, n = e.n_tok;
    const double* sc = scores + e.state_off;
    const int half = n / 2;
    if (half == 0) {  // no token is marked: every bit is 0
        if (tid == 0) flags[blockIdx.x] = 0;
    }
    // ---- the smallest key of the top half: ascending rank n - half, by radix selection from the top byte down
    if (tid == 0) {
        s_prefix = 0;
        s_rank = (uint32_t)(n - half);
        s_gt = 0;
        s_eq = 0;
    }
    for (int pass = 7; pass >= 0 && half > 0; --pass) {
        hist[tid] = 0;
        __syncthreads();
        const uint64_t hi_mask = pass == 7 ? 0ull : (~0ull << (8 * (pass + 1)));
        const uint64_t prefix = s_prefix;
        for (int i = tid; i < n; i += 256) {
            const uint64_t k = score_key(sc[i]);
            if ((k & hi_mask) == (prefix & hi_mask)) atomicAdd(&hist[(k >> (8 * pass)) & 255], 1u);
        }
        __syncthreads();
        if (tid == 0) {
            uint32_t cum = 0, rank = s_rank;
            int b = 0;
            for (; b < 255; ++b) {
                if (cum + hist[b] > rank) break;
                cum += hist[b];
            }
            s_rank = rank - cum;
            s_prefix = prefix | ((uint64_t)b << (8 * pass));
        }
        __syncthreads();
    }
    const uint64_t thr = s_prefix;
    if (half > 0) {
        uint32_t gt = 0, eq = 0;
        for (int i = tid; i < n; i += 256) {
            const uint64_t k = score_key(sc[i]);
            gt += k > thr;
            eq += k == thr;
        }
        atomicAdd(&s_gt, gt);
        atomicAdd(&s_eq, eq);
        __syncthreads();
        // all tokens at the threshold belong to the half, or the choice among them is the sorting routine's
        if (tid == 0) flags[blockIdx.x] = (s_eq == (uint32_t)half - s_gt) ? 0 : 1;
    }
    auto bit = [&](int i) -> uint32_t { return half > 0 && score_key(sc[i]) >= thr ? 1u : 0u; };
    // ---- the anchor point: bsz bits in `ones`
    const int blocks = n / bsz;
    for (int j = tid; j < bsz; j += 256) ones[j] = 0;
    __syncthreads();
    if (anchor_mode == pa::ANCHOR_MEAN) {  // majority bit per in-block position (kvcrush.cpp:57-69)
        for (int i = tid; i < blocks * bsz; i += 256)
            if (bit(i)) atomicAdd(&ones[i % bsz], 1u);
        __syncthreads();
        for (int j = tid; j < bsz; j += 256) ones[j] = 2 * ones[j] > (uint32_t)blocks ? 1u : 0u;
    } else {
        for (int j = tid; j < bsz; j += 256)
            ones[j] = anchor_mode == pa::ANCHOR_ZEROS ? 0u : anchor_mode == pa::ANCHOR_ONES ? 1u
                    : anchor_mode == pa::ANCHOR_ALTERNATING ? (uint32_t)(j & 1) : (uint32_t)host_anchors[e.anchor_off + j];
    }
    __syncthreads();
    // ---- Hamming distance of every block's bits to the anchor (kvcrush.cpp:84-111): a wave per block
    const int lane = tid & 63, wv = tid >> 6;
    for (int b = wv; b < blocks; b += 4) {
        uint32_t d = 0;
        for (int j = lane; j < bsz; j += 64) d += bit(b * bsz + j) != ones[j];
        for (int o = 32; o > 0; o >>= 1) d += __shfl_xor(d, o, 64);
        if (lane == 0) dist[e.dist_off + b] = (int32_t)d;
    }
}

constexpr int RKV_MAX_WINDOW = 32;

struct RkvEntry {        // one (sequence, layer) of a register call in ADAPTIVE_RKV mode
    int64_t src_off;     // first tracked score inside scores.<layer>
    int64_t state_off;   // first entry of this (slot, layer) in the score array
    int64_t hist_off;    // first entry of this (slot, layer)'s ring (window vectors of `cap` entries)
    int32_t new_len;
    int32_t rule;        // RULE_SKIP | RULE_INIT | RULE_ADD
    int32_t n;           // vectors in the ring, the new one included
    int32_t put;         // ring position that receives the new vector
    int32_t order[RKV_MAX_WINDOW];  // ring positions, oldest first
    int32_t lens[RKV_MAX_WINDOW];   // their lengths
};

// The new vector goes into the ring as it is (this mode pools after averaging); a first registration also
// becomes the tracked score.
__global__ __launch_bounds__(256) void evict_rkv_push_kernel(const RkvEntry* __restrict__ entries,
                                                             const float* const* __restrict__ layer_scores,
                                                             double* __restrict__ hist, double* __restrict__ scores,
                                                             int32_t layers, int64_t cap) {
    const int l = blockIdx.z;
    const RkvEntry& e = entries[(long)blockIdx.y * layers + l];
    if (e.rule == RULE_SKIP) return;
    const float* src = layer_scores[l] + e.src_off;
    double* dst = hist + e.hist_off + (int64_t)e.put * cap;
    for (int i = blockIdx.x * 256 + threadIdx.x; i < e.new_len; i += gridDim.x * 256) {
        const double v = (double)src[i];
        dst[i] = v;
        if (e.rule == RULE_INIT) scores[e.state_off + i] = v;
    }
}

// Tracked score = forward max-pool of the mean over the ring.  The sum runs oldest to newest and starts from
// the oldest vector's value where it has one, from zero past its end; shorter (older) vectors simply end.
__global__ __launch_bounds__(256) void evict_rkv_mean_pool_kernel(const RkvEntry* __restrict__ entries,
                                                                  const double* __restrict__ hist,
                                                                  double* __restrict__ scores, int32_t layers,
                                                                  int64_t cap, int32_t pool) {
#pragma clang fp contract(off)
    const int l = blockIdx.z;
    const RkvEntry& e = entries[(long)blockIdx.y * layers + l];
    if (e.rule != RULE_ADD) return;
    const double* ring = hist + e.hist_off;
    const int m = e.new_len;
    const double count = (double)e.n;
    for (int i = blockIdx.x * 256 + threadIdx.x; i < m; i += gridDim.x * 256) {
        const int eff = max(1, min(pool, m - i));
        double best = 0.0;
        for (int k = 0; k < eff; ++k) {
            const int t = i + k;
            double acc = t < e.lens[0] ? ring[(int64_t)e.order[0] * cap + t] : 0.0;
            for (int j = 1; j < e.n; ++j)
                if (t < e.lens[j]) acc += ring[(int64_t)e.order[j] * cap + t];
            const double mean = acc / count;
            best = k == 0 ? mean : (mean < best ? best : mean);
        }
        scores[e.state_off + i] = best;
    }
}

struct FiltEntry {       // one (sequence, layer) whose diversity set needs its filtered diversity
    const float* div;    // [n_blocks, n_blocks * block] registered diversity
    int64_t list_off;    // first entry in the in-set flags / output
    int32_t n_blocks;
    int32_t set_size;
};

// out[row] = (sum over the set's blocks, ascending, of (sum of the block's columns in this row)) / (set size * block).
// A block's columns are summed by one thread in column order, the blocks by thread 0 in block order: the
// association of a scalar evaluation.
__global__ __launch_bounds__(256) void evict_filtered_diversity_kernel(const FiltEntry* __restrict__ entries,
                                                                       const int32_t* __restrict__ in_set,
                                                                       double* __restrict__ out, int32_t bsz) {
#pragma clang fp contract(off)
    __shared__ double part[256];
    __shared__ int32_t has[256];
    const FiltEntry e = entries[blockIdx.x];
    const int row = blockIdx.y;
    if (row >= e.n_blocks) return;
    const float* r = e.div + (int64_t)row * e.n_blocks * bsz;
    const int32_t* flag = in_set + e.list_off;
    double acc = 0.0;
    for (int base = 0; base < e.n_blocks; base += 256) {
        const int b = base + threadIdx.x;
        const bool mine = b < e.n_blocks && flag[b] != 0;
        double p = 0.0;
        if (mine)
            for (int j = 0; j < bsz; ++j) p += (double)r[(int64_t)b * bsz + j];
        part[threadIdx.x] = p;
        has[threadIdx.x] = mine ? 1 : 0;
        __syncthreads();
        if (threadIdx.x == 0) {
            const int lim = min(256, e.n_blocks - base);
            for (int t = 0; t < lim; ++t)
                if (has[t]) acc += part[t];
        }
        __syncthreads();
    }
    if (threadIdx.x == 0) out[e.list_off + row] = acc / (double)((int64_t)e.set_size * bsz);
}

// Pinned host memory that only ever grows (allocated, never registered).
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
        std::memset(p, 0, want);  // the host's first touch of the pages happens here, not in the call that reads them
    }
    void release() {
        if (p) (void)hipHostFree(p);
        p = nullptr;
        cap = 0;
    }
    template <class T>
    T* as() const { return static_cast<T*>(p); }
};

struct DevBuf {
    void* p = nullptr;
    size_t cap = 0;
    void reserve(size_t bytes) {
        if (bytes <= cap) return;
        if (p) HIP_CHECK(hipFree(p));
        p = nullptr;
        cap = 0;
        HIP_CHECK(hipMalloc(&p, std::max<size_t>(bytes, 256)));
        cap = std::max<size_t>(bytes, 256);
    }
    void release() {
        if (p) (void)hipFree(p);
        p = nullptr;
        cap = 0;
    }
    template <class T>
    T* as() const { return static_cast<T*>(p); }
};

}  // namespace

struct pa_evictor {
    pa_evictor_config cfg{};
    bool has_areas = true;
    uint64_t ignore_blocks = 0;
    uint64_t evictable_size = 0;
    hipStream_t stream = nullptr;
    std::string error;
    double* scores = nullptr;
    unsigned long long* counters = nullptr;
    std::vector<uint64_t> len;          // [slot * L + layer]
    std::vector<uint64_t> snapkv_seen;  // [slot]
    DevBuf d_entries, d_ptrs, d_bscore, d_flags, d_list, d_filt, d_gather, d_gather_entries, d_copies;
    // pinned host staging: one buffer for what a call uploads, one for what it reads back; `staged` marks the end
    // of the last upload from h_up (the buffer may be refilled once it has passed)
    PinnedBuf h_up, h_back;
    hipEvent_t staged = nullptr;
    bool staged_pending = false;
    std::vector<uint8_t> slot_mark;     // [max_sequences] scratch of the duplicate-slot check
    // ADAPTIVE_RKV: ring of the last `window` score vectors per (slot, layer)
    double* hist = nullptr;
    std::vector<int32_t> ring_len;    // [(slot * L + layer) * window + position]
    std::vector<int32_t> ring_head;   // [slot * L + layer] position of the oldest vector
    std::vector<int32_t> ring_count;  // [slot * L + layer]
    // diversity registered for the coming eviction, copied into library memory: per slot, layer l's matrix
    // starts at div_off[slot][l] floats
    std::vector<DevBuf> div_buf;                 // [slot]
    std::vector<std::vector<uint64_t>> div_off;  // [slot][L + 1]; empty = nothing registered
    std::vector<pa::KvCrushSelector> crush;      // [slot]

    bool rkv() const { return cfg.aggregation_mode == PA_AGG_ADAPTIVE_RKV; }
    uint64_t W() const { return cfg.adaptive_rkv_window_size; }
    int64_t hist_off(int32_t slot, uint64_t layer) const {
        return (int64_t)(((uint64_t)slot * L() + layer) * W() * cfg.max_tracked_tokens);
    }
    void clear_ring(int32_t slot, uint64_t layer) { ring_count[(uint64_t)slot * L() + layer] = 0; }
    uint64_t L() const { return cfg.num_decoder_layers; }
    uint64_t max_after() const { return cfg.max_cache_size + cfg.block_size - 1; }
    int64_t state_off(int32_t slot, uint64_t layer) const {
        return (int64_t)(((uint64_t)slot * L() + layer) * cfg.max_tracked_tokens);
    }
    // get_evictable_block_range, cache_eviction.cpp:416-424
    bool range(int32_t slot, uint64_t layer, uint64_t* b, uint64_t* e) const {
        const uint64_t cur = cfg.start_size + len[(uint64_t)slot * L() + layer];
        if (!has_areas || cur <= max_after()) { *b = 0; *e = 0; return false; }
        *b = cfg.start_size / cfg.block_size;
        *e = cur / cfg.block_size - cfg.recent_size / cfg.block_size;
        return true;
    }
    // get_num_blocks_to_evict, cache_eviction.cpp:448-455
    uint64_t num_to_evict(uint64_t n_evictable) const {
        const uint64_t keep = (evictable_size + cfg.block_size - 1) / cfg.block_size;
        return n_evictable < keep ? 0 : n_evictable - keep;
    }
};

namespace {

template <class Fn>
int32_t guarded(pa_evictor* ev, Fn&& fn) {
    auto set = [&](const std::string& m) { if (ev) ev->error = m; else g_evict_error = m; };
    try {
        fn();
        return PA_OK;
    } catch (const StatusError& e) {
        set(e.what());
        return e.code;
    } catch (const std::bad_alloc&) {
        set("host allocation failed");
        return PA_NOT_ALLOCATED;
    } catch (const std::exception& e) {
        set(e.what());
        return PA_UNKNOWN_EXCEPTION;
    } catch (...) {
        set("unknown exception");
        return PA_UNKNOWN_EXCEPTION;
    }
}

void check_slot(const pa_evictor* ev, int32_t slot) {
    PA_REQUIRE(slot >= 0 && (uint64_t)slot < ev->cfg.max_sequences, PA_OUT_OF_BOUNDS, "slot out of range");
}

pa_evictor* make(const pa_evictor_config* cfg, bool areas, uint64_t ignore_blocks) {
    PA_REQUIRE(cfg, PA_INVALID_C_PARAM, "config is null");
    PA_REQUIRE(cfg->block_size > 0, PA_PARAMETER_MISMATCH, "block_size must be non-zero");
    PA_REQUIRE(cfg->num_decoder_layers > 0, PA_PARAMETER_MISMATCH, "num_decoder_layers must be non-zero");
    PA_REQUIRE(cfg->aggregation_mode == PA_AGG_SUM || cfg->aggregation_mode == PA_AGG_NORM_SUM ||
                   cfg->aggregation_mode == PA_AGG_ADAPTIVE_RKV,
               PA_PARAMETER_MISMATCH, "unknown aggregation mode");
    if (cfg->aggregation_mode == PA_AGG_ADAPTIVE_RKV) {
        PA_REQUIRE(cfg->adaptive_rkv_window_size >= 1 && cfg->adaptive_rkv_window_size <= (uint64_t)RKV_MAX_WINDOW,
                   PA_NOT_IMPLEMENTED, "AdaptiveRKVConfig.window_size must lie in [1, 32]");
    }
    PA_REQUIRE(cfg->kvcrush_anchor_point_mode >= pa::ANCHOR_RANDOM && cfg->kvcrush_anchor_point_mode <= pa::ANCHOR_ALTERNATING,
               PA_PARAMETER_MISMATCH, "Invalid anchor point type");
    PA_REQUIRE(cfg->max_sequences > 0 && cfg->max_tracked_tokens > 0, PA_PARAMETER_MISMATCH,
               "max_sequences and max_tracked_tokens must be non-zero");
    PA_REQUIRE(cfg->max_tracked_tokens <= (uint64_t)INT32_MAX, PA_OUT_OF_BOUNDS, "max_tracked_tokens too large");
    if (areas) {
        PA_REQUIRE(cfg->start_size, PA_PARAMETER_MISMATCH, "CacheEvictionConfig.start_size must be non-zero");
        PA_REQUIRE(cfg->recent_size, PA_PARAMETER_MISMATCH, "CacheEvictionConfig.recent_size must be non-zero");
        PA_REQUIRE(cfg->max_cache_size, PA_PARAMETER_MISMATCH, "CacheEvictionConfig.max_cache_size must be non-zero");
        PA_REQUIRE(cfg->max_cache_size > cfg->start_size + cfg->recent_size, PA_PARAMETER_MISMATCH,
                   "CacheEvictionConfig.max_cache_size must be larger than CacheEvictionConfig.start_size + "
                   "CacheEvictionConfig.recent_size");
        PA_REQUIRE(cfg->start_size % cfg->block_size == 0, PA_PARAMETER_MISMATCH,
                   "CacheEvictionConfig.start_size in tokens must be a multiple of block size");
        PA_REQUIRE(cfg->recent_size % cfg->block_size == 0, PA_PARAMETER_MISMATCH,
                   "CacheEvictionConfig.recent_size in tokens must be a multiple of block size");
        PA_REQUIRE(cfg->max_cache_size % cfg->block_size == 0, PA_PARAMETER_MISMATCH,
                   "CacheEvictionConfig.max_cache_size in tokens must be a multiple of block size");
    }
    int ndev = 0;
    HIP_CHECK(hipGetDeviceCount(&ndev));
    PA_REQUIRE(cfg->device >= 0 && cfg->device < ndev, PA_OUT_OF_BOUNDS, "no such HIP device");
    HIP_CHECK(hipSetDevice(cfg->device));
    pa_evictor* ev = new pa_evictor();
    ev->cfg = *cfg;
    ev->has_areas = areas;
    ev->ignore_blocks = areas ? cfg->start_size / cfg->block_size : ignore_blocks;
    ev->evictable_size = areas ? cfg->max_cache_size - cfg->start_size - cfg->recent_size : 0;
    ev->stream = static_cast<hipStream_t>(cfg->stream);
    const size_t n = (size_t)cfg->max_sequences * cfg->num_decoder_layers * cfg->max_tracked_tokens;
    hipError_t e1 = hipMalloc(reinterpret_cast<void**>(&ev->scores), n * sizeof(double));
    hipError_t e2 = e1 == hipSuccess ? hipMalloc(reinterpret_cast<void**>(&ev->counters), n * sizeof(unsigned long long))
                                     : e1;
    hipError_t e3 = hipSuccess;
    if (e2 == hipSuccess && ev->rkv())
        e3 = hipMalloc(reinterpret_cast<void**>(&ev->hist), n * cfg->adaptive_rkv_window_size * sizeof(double));
    if (e1 != hipSuccess || e2 != hipSuccess || e3 != hipSuccess) {
        (void)hipGetLastError();
        if (ev->scores) (void)hipFree(ev->scores);
        if (ev->counters) (void)hipFree(ev->counters);
        delete ev;
        throw StatusError(PA_NOT_ALLOCATED, "not enough device memory for the eviction state");
    }
    if (hipEventCreateWithFlags(&ev->staged, hipEventDisableTiming) != hipSuccess) {
        (void)hipGetLastError();
        (void)hipFree(ev->scores);
        (void)hipFree(ev->counters);
        if (ev->hist) (void)hipFree(ev->hist);
        delete ev;
        throw StatusError(PA_GENERAL_ERROR, "could not create the staging event");
    }
    ev->slot_mark.assign(cfg->max_sequences, 0);
    const size_t pairs = (size_t)cfg->max_sequences * cfg->num_decoder_layers;
    try {  // what a call over every slot uploads and reads back at least, so that the first call does not allocate it
        const size_t up = ((size_t)cfg->num_decoder_layers * sizeof(float*) + 15) / 16 * 16 + pairs * sizeof(RegEntry);
        ev->h_up.reserve(up);
        ev->d_entries.reserve(pairs * std::max(sizeof(RegEntry), sizeof(SelEntry)));
        ev->d_ptrs.reserve((size_t)cfg->num_decoder_layers * sizeof(float*));
        // (block lists of a whole-context eviction of every pair: 1 / (4 * block_size) of the tracked scores' size)
        const size_t lists = pairs * std::max<size_t>(1, (size_t)(cfg->max_tracked_tokens / cfg->block_size)) * sizeof(int32_t);
        ev->d_list.reserve(lists);
        ev->h_back.reserve(lists);
    } catch (...) {
        (void)hipFree(ev->scores);
        (void)hipFree(ev->counters);
        if (ev->hist) (void)hipFree(ev->hist);
        ev->h_up.release();
        ev->d_entries.release();
        ev->d_ptrs.release();
        ev->d_list.release();
        (void)hipEventDestroy(ev->staged);
        delete ev;
        throw;
    }
    ev->len.assign(pairs, 0);
    ev->snapkv_seen.assign(cfg->max_sequences, 0);
    if (ev->rkv()) {
        ev->ring_len.assign(pairs * cfg->adaptive_rkv_window_size, 0);
        ev->ring_head.assign(pairs, 0);
        ev->ring_count.assign(pairs, 0);
    }
    ev->div_buf.resize(cfg->max_sequences);
    ev->div_off.resize(cfg->max_sequences);
    ev->crush.resize(cfg->max_sequences);
    for (auto& c : ev->crush)
        c.init(cfg->kvcrush_budget, cfg->kvcrush_anchor_point_mode, cfg->kvcrush_rng_seed, cfg->block_size);
    return ev;
}

void upload(pa_evictor* ev, DevBuf& buf, const void* src, size_t bytes) {
    buf.reserve(bytes);
    HIP_CHECK(hipMemcpyAsync(buf.p, src, bytes, hipMemcpyHostToDevice, ev->stream));
    HIP_CHECK(hipStreamSynchronize(ev->stream));
}

// Pinned staging of what a call uploads: stage_begin hands out the buffer once the previous call's copy out of it has
// passed, stage_copy enqueues a copy of a piece of it, stage_end marks the end of the call's copies.  Nothing waits for
// the copies themselves: the kernels that read them follow on the same stream.
uint8_t* stage_begin(pa_evictor* ev, size_t bytes) {
    if (ev->staged_pending) {
        HIP_CHECK(hipEventSynchronize(ev->staged));
        ev->staged_pending = false;
    }
    ev->h_up.reserve(bytes);
    return ev->h_up.as<uint8_t>();
}
void stage_copy(pa_evictor* ev, DevBuf& dst, size_t stage_off, size_t bytes) {
    dst.reserve(bytes);
    HIP_CHECK(hipMemcpyAsync(dst.p, ev->h_up.as<uint8_t>() + stage_off, bytes, hipMemcpyHostToDevice, ev->stream));
}
void stage_end(pa_evictor* ev) {
    HIP_CHECK(hipEventRecord(ev->staged, ev->stream));
    ev->staged_pending = true;
}

// Every slot of a call is in range and listed once.
void check_slots(pa_evictor* ev, int32_t B, const int32_t* slots) {
    bool twice = false;
    int32_t i = 0;
    for (; i < B; ++i) {
        if (slots[i] < 0 || (uint64_t)slots[i] >= ev->cfg.max_sequences) break;
        twice = twice || ev->slot_mark[slots[i]];
        ev->slot_mark[slots[i]] = 1;
    }
    for (int32_t j = 0; j < i; ++j) ev->slot_mark[slots[j]] = 0;
    PA_REQUIRE(i == B, PA_OUT_OF_BOUNDS, "slot out of range");
    PA_REQUIRE(!twice, PA_PARAMETER_MISMATCH, "slot listed twice");
}

// Runs compaction for prepared entries whose evicted lists are already in d_list.
void compact(pa_evictor* ev, const std::vector<SelEntry>& entries) {
    hipLaunchKernelGGL(evict_compact_kernel, dim3((unsigned)entries.size()), dim3(256), 0, ev->stream,
                       ev->d_entries.as<SelEntry>(), ev->d_list.as<int32_t>(), ev->scores, ev->counters,
                       (int32_t)ev->cfg.block_size, ev->cfg.aggregation_mode == PA_AGG_NORM_SUM ? 1 : 0);
    HIP_CHECK(hipGetLastError());
}

// ADAPTIVE_RKV branch of register_new_token_scores (cache_eviction.cpp:113-117, 129-141, 162-181).
void register_rkv(pa_evictor* ev, int32_t B, const int32_t* slots, const float* const* scores_per_layer,
                  const int64_t* offsets, const uint64_t* num_snapkv, const std::vector<uint64_t>& seen) {
    const uint64_t L = ev->L(), bsz = ev->cfg.block_size, window = ev->cfg.snapkv_window_size, W = ev->W();
    std::vector<RkvEntry> entries((size_t)B * L);
    int32_t longest = 0;
    bool any_add = false;
    for (int32_t i = 0; i < B; ++i) {
        const uint64_t n = (uint64_t)(offsets[i + 1] - offsets[i]);
        const uint64_t ns = num_snapkv ? num_snapkv[i] : 0;
        for (uint64_t l = 0; l < L; ++l) {
            RkvEntry& e = entries[(size_t)i * L + l];
            std::memset(&e, 0, sizeof(e));
            e.rule = RULE_SKIP;
            if (n <= ev->ignore_blocks * bsz) continue;
            const uint64_t m = n - ev->ignore_blocks * bsz;
            const uint64_t sl = (uint64_t)slots[i] * L + l;
            PA_REQUIRE(m <= ev->cfg.max_tracked_tokens, PA_OUT_OF_BOUNDS, "score vector longer than max_tracked_tokens");
            e.src_off = offsets[i] + (int64_t)(ev->ignore_blocks * bsz);
            e.state_off = ev->state_off(slots[i], l);
            e.hist_off = ev->hist_off(slots[i], l);
            e.new_len = (int32_t)m;
            int32_t head = ev->ring_head[sl], count = ev->ring_count[sl];
            if (ev->len[sl] == 0) {
                if (window != 0 && ns == 0) continue;  // SnapKV window not reached yet
                PA_REQUIRE(count == 0, PA_GENERAL_ERROR, "score history present without tracked scores");
                e.rule = RULE_INIT;
            } else {
                if (count > 0) {
                    const int32_t newest = ev->ring_len[sl * W + (uint64_t)((head + count - 1) % (int32_t)W)];
                    PA_REQUIRE((int32_t)m >= newest, PA_PARAMETER_MISMATCH,
                               "registered scores are shorter than the ones registered before");
                }
                e.rule = RULE_ADD;
                any_add = true;
                if (count >= (int32_t)W) {  // the oldest vector leaves
                    head = (head + 1) % (int32_t)W;
                    --count;
                }
            }
            e.put = (head + count) % (int32_t)W;
            e.n = count + 1;
            for (int32_t j = 0; j < count; ++j) {
                e.order[j] = (head + j) % (int32_t)W;
                e.lens[j] = ev->ring_len[sl * W + (uint64_t)e.order[j]];
            }
            e.order[count] = e.put;
            e.lens[count] = e.new_len;
            longest = std::max(longest, e.new_len);
        }
    }
    HIP_CHECK(hipSetDevice(ev->cfg.device));
    if (longest > 0) {
        upload(ev, ev->d_entries, entries.data(), entries.size() * sizeof(RkvEntry));
        upload(ev, ev->d_ptrs, scores_per_layer, L * sizeof(float*));
        const dim3 grid((unsigned)std::min(pa::ceil_div(longest, 256), 64), (unsigned)B, (unsigned)L);
        hipLaunchKernelGGL(evict_rkv_push_kernel, grid, dim3(256), 0, ev->stream, ev->d_entries.as<RkvEntry>(),
                           ev->d_ptrs.as<const float*>(), ev->hist, ev->scores, (int32_t)L,
                           (int64_t)ev->cfg.max_tracked_tokens);
        if (any_add)
            hipLaunchKernelGGL(evict_rkv_mean_pool_kernel, grid, dim3(256), 0, ev->stream, ev->d_entries.as<RkvEntry>(),
                               ev->hist, ev->scores, (int32_t)L, (int64_t)ev->cfg.max_tracked_tokens,
                               (int32_t)ev->cfg.max_pool_window_size);
        HIP_CHECK(hipGetLastError());
        HIP_CHECK(hipStreamSynchronize(ev->stream));
    }
    for (int32_t i = 0; i < B; ++i) {
        ev->snapkv_seen[slots[i]] = seen[i];
        for (uint64_t l = 0; l < L; ++l) {
            const RkvEntry& e = entries[(size_t)i * L + l];
            if (e.rule == RULE_SKIP) continue;
            const uint64_t sl = (uint64_t)slots[i] * L + l;
            ev->len[sl] = (uint64_t)e.new_len;
            ev->ring_head[sl] = e.order[0];
            ev->ring_count[sl] = e.n;
            ev->ring_len[sl * W + (uint64_t)e.put] = e.new_len;
        }
    }
}

}  // namespace

extern "C" {

int32_t pa_evictor_create(const pa_evictor_config* cfg, pa_evictor** out) {
    return guarded(nullptr, [&] {
        PA_REQUIRE(out, PA_INVALID_C_PARAM, "out is null");
        *out = nullptr;
        *out = make(cfg, true, 0);
    });
}

int32_t pa_score_manager_create(const pa_evictor_config* cfg, uint64_t ignore_first_n_blocks, pa_evictor** out) {
    return guarded(nullptr, [&] {
        PA_REQUIRE(out, PA_INVALID_C_PARAM, "out is null");
        *out = nullptr;
        *out = make(cfg, false, ignore_first_n_blocks);
    });
}

void pa_evictor_destroy(pa_evictor* ev) {
    if (!ev) return;
    (void)hipSetDevice(ev->cfg.device);
    (void)hipStreamSynchronize(ev->stream);
    if (ev->scores) (void)hipFree(ev->scores);
    if (ev->counters) (void)hipFree(ev->counters);
    if (ev->hist) (void)hipFree(ev->hist);
    for (auto& b : ev->div_buf) b.release();
    ev->d_filt.release();
    ev->d_copies.release();
    ev->d_entries.release();
    ev->d_ptrs.release();
    ev->d_bscore.release();
    ev->d_flags.release();
    ev->d_list.release();
    ev->d_gather.release();
    ev->d_gather_entries.release();
    ev->h_up.release();
    ev->h_back.release();
    if (ev->staged) (void)hipEventDestroy(ev->staged);
    delete ev;
}

const char* pa_evictor_last_error(const pa_evictor* ev) { return ev ? ev->error.c_str() : g_evict_error.c_str(); }

int32_t pa_evictor_reset_slot(pa_evictor* ev, int32_t slot) {
    if (!ev) return PA_INVALID_C_PARAM;
    return guarded(ev, [&] {
        check_slot(ev, slot);
        for (uint64_t l = 0; l < ev->L(); ++l) {
            ev->len[(uint64_t)slot * ev->L() + l] = 0;
            if (ev->rkv()) ev->clear_ring(slot, l);
        }
        ev->snapkv_seen[slot] = 0;
        ev->div_off[slot].clear();
        // a new sequence gets a new KVCrushAlgorithm, hence a freshly seeded generator (cache_eviction.cpp:286)
        ev->crush[slot].init(ev->cfg.kvcrush_budget, ev->cfg.kvcrush_anchor_point_mode, ev->cfg.kvcrush_rng_seed,
                             ev->cfg.block_size);
    });
}

int32_t pa_evictor_register_scores(pa_evictor* ev, int32_t B, const int32_t* slots,
                                   const float* const* scores_per_layer, const int64_t* offsets,
                                   const uint64_t* num_snapkv) {
    if (!ev) return PA_INVALID_C_PARAM;
    return guarded(ev, [&] {
        PA_REQUIRE(B > 0 && slots && scores_per_layer && offsets, PA_INVALID_C_PARAM, "null argument");
        const uint64_t L = ev->L(), bsz = ev->cfg.block_size, window = ev->cfg.snapkv_window_size;
        const bool norm = ev->cfg.aggregation_mode == PA_AGG_NORM_SUM;
        for (uint64_t l = 0; l < L; ++l)
            PA_REQUIRE(scores_per_layer[l] && (reinterpret_cast<uintptr_t>(scores_per_layer[l]) & 3) == 0, PA_INVALID_C_PARAM,
                       "null scores pointer, or one that is not a multiple of 4 bytes");
        // validate everything before touching state
        std::vector<uint64_t> seen(B);
        check_slots(ev, B, slots);
        for (int32_t i = 0; i < B; ++i) {
            PA_REQUIRE(offsets[i + 1] >= offsets[i], PA_PARAMETER_MISMATCH, "offsets must be non-decreasing");
            const uint64_t ns = num_snapkv ? num_snapkv[i] : 0;
            uint64_t s = ev->snapkv_seen[slots[i]];
            if (s < window) {
                PA_REQUIRE(ns + s <= window, PA_PARAMETER_MISMATCH,
                           "Total number of aggregated SnapKV scores during prefill phase may not be larger than the "
                           "configured SnapKV window size");
                s += ns;
            }
            seen[i] = s;
        }
        if (ev->rkv()) {
            register_rkv(ev, B, slots, scores_per_layer, offsets, num_snapkv, seen);
            return;
        }
        std::vector<RegEntry> entries((size_t)B * L);
        int32_t longest = 0;
        for (int32_t i = 0; i < B; ++i) {
            const uint64_t n = (uint64_t)(offsets[i + 1] - offsets[i]);
            const uint64_t ns = num_snapkv ? num_snapkv[i] : 0;
            for (uint64_t l = 0; l < L; ++l) {
                RegEntry& e = entries[(size_t)i * L + l];
                e = RegEntry{0, 0, 0, 0, RULE_SKIP, 0};
                if (n <= ev->ignore_blocks * bsz) continue;
                const uint64_t m = n - ev->ignore_blocks * bsz;
                const uint64_t old = ev->len[(uint64_t)slots[i] * L + l];
                PA_REQUIRE(m <= ev->cfg.max_tracked_tokens, PA_OUT_OF_BOUNDS,
                           "score vector longer than max_tracked_tokens");
                e.src_off = offsets[i] + (int64_t)(ev->ignore_blocks * bsz);
                e.state_off = ev->state_off(slots[i], l);
                e.old_len = (int32_t)old;
                e.new_len = (int32_t)m;
                if (old == 0) {
                    if (window != 0 && ns == 0) { e.rule = RULE_SKIP; continue; }
                    if (window == 0) {
                        e.rule = RULE_INIT;
                    } else {
                        PA_REQUIRE(m >= ns, PA_PARAMETER_MISMATCH, "fewer scores than SnapKV scores");
                        e.rule = RULE_INIT_SNAPKV;
                        e.snap = (int32_t)ns;
                    }
                } else {
                    PA_REQUIRE(m >= old, PA_PARAMETER_MISMATCH, "registered scores are shorter than the tracked ones");
                    if (window == 0 || seen[i] == window) {
                        e.rule = RULE_ADD;
                    } else {
                        PA_REQUIRE(m >= seen[i], PA_PARAMETER_MISMATCH, "fewer scores than registered SnapKV scores");
                        e.rule = RULE_ADD_SNAPKV;
                        e.snap = (int32_t)seen[i];
                    }
                }
                longest = std::max(longest, e.new_len);
            }
        }
        HIP_CHECK(hipSetDevice(ev->cfg.device));
        if (longest > 0) {
            // one pinned staging buffer (layer pointers | entries), two copies, one launch; nothing waits: whatever
            // reads the state later follows on the same stream
            const size_t ptr_bytes = (L * sizeof(float*) + 15) & ~(size_t)15, ent_bytes = entries.size() * sizeof(RegEntry);
            uint8_t* st = stage_begin(ev, ptr_bytes + ent_bytes);
            std::memcpy(st, scores_per_layer, L * sizeof(float*));
            std::memcpy(st + ptr_bytes, entries.data(), ent_bytes);
            stage_copy(ev, ev->d_ptrs, 0, L * sizeof(float*));
            stage_copy(ev, ev->d_entries, ptr_bytes, ent_bytes);
            stage_end(ev);
            dim3 grid((unsigned)std::min(pa::ceil_div(longest, 256), 64), (unsigned)B, (unsigned)L);
            hipLaunchKernelGGL(evict_register_kernel, grid, dim3(256), 0, ev->stream, ev->d_entries.as<RegEntry>(),
                               ev->d_ptrs.as<const float*>(), ev->scores, ev->counters, (int32_t)L,
                               (int32_t)ev->cfg.max_pool_window_size, norm ? 1 : 0);
            HIP_CHECK(hipGetLastError());
        }
        for (int32_t i = 0; i < B; ++i) {
            ev->snapkv_seen[slots[i]] = seen[i];
            for (uint64_t l = 0; l < L; ++l) {
                const RegEntry& e = entries[(size_t)i * L + l];
                if (e.rule != RULE_SKIP) ev->len[(uint64_t)slots[i] * L + l] = (uint64_t)e.new_len;
            }
        }
    });
}

int32_t pa_evictor_register_block_diversity(pa_evictor* ev, int32_t B, const int32_t* slots,
                                            const float* const* diversity_per_layer, const int64_t* offsets) {
    if (!ev) return PA_INVALID_C_PARAM;
    return guarded(ev, [&] {
        PA_REQUIRE(B > 0 && slots && diversity_per_layer && offsets, PA_INVALID_C_PARAM, "null argument");
        const uint64_t L = ev->L();
        for (uint64_t l = 0; l < L; ++l) PA_REQUIRE(diversity_per_layer[l], PA_INVALID_C_PARAM, "null diversity pointer");
        check_slots(ev, B, slots);
        for (int32_t i = 0; i < B; ++i) {
            PA_REQUIRE(offsets[i + 1] >= offsets[i], PA_PARAMETER_MISMATCH, "offsets must be non-decreasing");
            PA_REQUIRE(ev->div_off[slots[i]].empty(), PA_PARAMETER_MISMATCH,
                       "CacheEvictionAlgorithm already has block_diversity, must evict before new diversity is registered");
            PA_REQUIRE((uint64_t)(offsets[i + 1] - offsets[i]) % ev->cfg.block_size == 0, PA_PARAMETER_MISMATCH,
                       "diversity size must be a multiple of the block size");
        }
        HIP_CHECK(hipSetDevice(ev->cfg.device));
        // one launch copies every (sequence, layer) matrix; the per-sequence buffers only ever grow
        const size_t bytes = (size_t)B * L * sizeof(CopyEntry);
        CopyEntry* copies = reinterpret_cast<CopyEntry*>(stage_begin(ev, bytes));
        int64_t longest = 0;
        for (int32_t i = 0; i < B; ++i) {
            const uint64_t n = (uint64_t)(offsets[i + 1] - offsets[i]);
            DevBuf& buf = ev->div_buf[slots[i]];
            buf.reserve(std::max<uint64_t>(1, n * L) * sizeof(float));
            for (uint64_t l = 0; l < L; ++l)
                copies[(size_t)i * L + l] = CopyEntry{diversity_per_layer[l] + offsets[i], buf.as<float>() + l * n, (int64_t)n};
            longest = std::max<int64_t>(longest, (int64_t)n);
        }
        if (longest > 0) {
            stage_copy(ev, ev->d_copies, 0, bytes);
            stage_end(ev);
            const unsigned gx = (unsigned)std::max<int64_t>(1, std::min<int64_t>((longest + 4095) / 4096, 256));
            hipLaunchKernelGGL(evict_copy_kernel, dim3((unsigned)((size_t)B * L), gx), dim3(256), 0, ev->stream,
                               ev->d_copies.as<CopyEntry>());
            HIP_CHECK(hipGetLastError());
        }
        for (int32_t i = 0; i < B; ++i) {
            const uint64_t n = (uint64_t)(offsets[i + 1] - offsets[i]);
            std::vector<uint64_t>& off = ev->div_off[slots[i]];
            off.resize(L + 1);
            for (uint64_t l = 0; l <= L; ++l) off[l] = l * n;
        }
    });
}

int32_t pa_evictor_evict(pa_evictor* ev, int32_t B, const int32_t* slots, int32_t* counts, int32_t* blocks,
                         int32_t max_per_entry) {
    if (!ev) return PA_INVALID_C_PARAM;
    return guarded(ev, [&] {
        PA_REQUIRE(B > 0 && slots && counts && blocks && max_per_entry >= 0, PA_INVALID_C_PARAM, "null argument");
        PA_REQUIRE(ev->has_areas, PA_PARAMETER_MISMATCH, "a bare score manager has no eviction areas");
        const uint64_t L = ev->L(), bsz = ev->cfg.block_size;
        const bool rkv = ev->rkv();
        bool crush = !rkv && ev->cfg.kvcrush_budget > 0;  // (below: and only where enough blocks are chosen)
        std::vector<SelEntry> entries((size_t)B * L);
        int64_t list_total = 0, k_total = 0;
        int32_t most_blocks_any = 0, most_k = 0;
        bool any = false;
        check_slots(ev, B, slots);
        for (int32_t i = 0; i < B; ++i) {
            for (uint64_t l = 0; l < L; ++l) {
                SelEntry& e = entries[(size_t)i * L + l];
                e = SelEntry{ev->state_off(slots[i], l), list_total, (int32_t)ev->len[(uint64_t)slots[i] * L + l], 0, 0, 0};
                uint64_t rb, re;
                if (ev->range(slots[i], l, &rb, &re)) {
                    e.n_blocks = (int32_t)(re - rb);
                    if (rkv) {  // cache_eviction.cpp:331-336
                        const std::vector<uint64_t>& off = ev->div_off[slots[i]];
                        PA_REQUIRE(!off.empty(), PA_PARAMETER_MISMATCH,
                                   "Token diversity must be registered before each eviction in the Adaptive R-KV scenario");
                        const uint64_t want = (re - rb) * (re - rb) * bsz;
                        PA_REQUIRE(off[1] - off[0] == want, PA_PARAMETER_MISMATCH,
                                   "Diversity score size mismatch - registered " + std::to_string(off[1] - off[0]) +
                                       " diversity scores, but expected " + std::to_string(want));
                        any = any || e.n_blocks > 0;
                    } else {
                        e.k = (int32_t)ev->num_to_evict(re - rb);
                        PA_REQUIRE(e.k <= max_per_entry, PA_OUT_OF_BOUNDS, "more evicted blocks than the output holds");
                        any = any || e.k > 0;
                        e.out_off = (int32_t)k_total;
                        k_total += e.k;
                        PA_REQUIRE(k_total <= INT32_MAX, PA_OUT_OF_BOUNDS, "too many evicted blocks for one call");
                        if (e.k > 0) most_blocks_any = std::max(most_blocks_any, e.n_blocks);
                        most_k = std::max(most_k, e.k);
                    }
                    list_total += e.n_blocks;
                }
            }
        }
        // lists: per pair at list_off (one entry per evictable block) or, packed, at out_off (one per evicted block)
        auto finish = [&](const int32_t* lists, bool packed) {
            const int32_t shift = (int32_t)(ev->cfg.start_size / bsz);
            for (int32_t i = 0; i < B; ++i) {
                for (uint64_t l = 0; l < L; ++l) {
                    const SelEntry& e = entries[(size_t)i * L + l];
                    counts[(size_t)i * L + l] = e.k;
                    const int32_t* mine = lists + (packed ? (size_t)e.out_off : (size_t)e.list_off);
                    for (int32_t p = 0; p < e.k; ++p)
                        blocks[((size_t)i * L + l) * max_per_entry + p] = mine[p] + shift;
                    ev->len[(uint64_t)slots[i] * L + l] -= (uint64_t)e.k * bsz;
                    if (rkv && e.k > 0) ev->clear_ring(slots[i], l);  // remove_scores drops the history, :50
                }
                ev->div_off[slots[i]].clear();  // :407
            }
        };
        if (!any) {
            finish(nullptr, false);
            return;
        }
        if (crush) {  // cache_eviction.cpp:365-366: representatives stay only where at least `budget` blocks were chosen
            crush = false;
            for (const SelEntry& e : entries) crush = crush || (e.k > 0 && (uint64_t)e.k >= ev->cfg.kvcrush_budget);
        }
        HIP_CHECK(hipSetDevice(ev->cfg.device));
        const int32_t norm = ev->cfg.aggregation_mode == PA_AGG_NORM_SUM ? 1 : 0;
        const size_t fused_lds = select_lds_bytes(most_blocks_any, (int64_t)bsz, most_k);
        if (!rkv && !crush && fused_lds <= 150 * 1024) {
            // the plain modes: one upload, one launch (scores, selection, list, removal), one read-back
            const size_t ent_bytes = entries.size() * sizeof(SelEntry);
            uint8_t* st = stage_begin(ev, ent_bytes);
            std::memcpy(st, entries.data(), ent_bytes);
            stage_copy(ev, ev->d_entries, 0, ent_bytes);
            stage_end(ev);
            ev->d_list.reserve((size_t)k_total * sizeof(int32_t));
            ev->h_back.reserve((size_t)k_total * sizeof(int32_t));
            HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(evict_select_compact_kernel),
                                          hipFuncAttributeMaxDynamicSharedMemorySize, (int)fused_lds));
            hipLaunchKernelGGL(evict_select_compact_kernel, dim3((unsigned)entries.size()), dim3(256), fused_lds, ev->stream,
                               ev->d_entries.as<SelEntry>(), ev->scores, ev->counters, ev->d_list.as<int32_t>(),
                               (int32_t)bsz, norm, most_blocks_any);
            HIP_CHECK(hipGetLastError());
            HIP_CHECK(hipMemcpyAsync(ev->h_back.p, ev->d_list.p, (size_t)k_total * sizeof(int32_t), hipMemcpyDeviceToHost,
                                     ev->stream));
            HIP_CHECK(hipStreamSynchronize(ev->stream));
            finish(ev->h_back.as<int32_t>(), true);
            return;
        }
        upload(ev, ev->d_entries, entries.data(), entries.size() * sizeof(SelEntry));
        ev->d_bscore.reserve((size_t)list_total * sizeof(double));
        ev->d_flags.reserve((size_t)list_total * sizeof(int32_t));
        ev->d_list.reserve((size_t)list_total * sizeof(int32_t));
        const dim3 grid((unsigned)entries.size()), block(256);
        hipLaunchKernelGGL(evict_block_score_kernel, grid, block, 0, ev->stream, ev->d_entries.as<SelEntry>(),
                           ev->scores, ev->counters, ev->d_bscore.as<double>(), (int32_t)bsz, norm);
        HIP_CHECK(hipGetLastError());
        std::vector<int32_t> lists((size_t)list_total);
        bool lists_on_device = false;
        if (rkv) {
            // the choice among a few hundred blocks runs on the host (cache_eviction.cpp:329-362)
            std::vector<double> bscore((size_t)list_total);
            HIP_CHECK(hipMemcpyAsync(bscore.data(), ev->d_bscore.p, bscore.size() * sizeof(double), hipMemcpyDeviceToHost,
                                     ev->stream));
            HIP_CHECK(hipStreamSynchronize(ev->stream));
            const pa::RkvBlockCalculator calc{ev->cfg.adaptive_rkv_attention_mass, (size_t)bsz};
            const size_t max_keep = ev->evictable_size / bsz;
            std::vector<std::set<size_t>> sets(entries.size());
            std::vector<size_t> left(entries.size(), 0);
            std::vector<int32_t> in_set((size_t)list_total, 0);
            std::vector<FiltEntry> filt;
            int32_t most_blocks = 0;
            // (the entries are independent: host threads share the two loops over them)
            pa::parallel_items(entries.size(), entries.size() / 64 + 1, [&](size_t x) {
                const SelEntry& e = entries[x];
                if (e.n_blocks <= 0) return;
                size_t kept = 0;
                sets[x] = calc.diversity_block_set(max_keep, bscore.data() + e.list_off, (size_t)e.n_blocks, &kept);
                left[x] = max_keep - kept;
                if (left[x] == 0) return;
                PA_REQUIRE(left[x] <= sets[x].size(), PA_GENERAL_ERROR,
                           "more blocks left to fill than the diversity set holds");
                for (size_t b : sets[x]) in_set[(size_t)e.list_off + b] = 1;
            });
            for (size_t x = 0; x < entries.size(); ++x) {
                const SelEntry& e = entries[x];
                if (e.n_blocks <= 0 || left[x] == 0) continue;
                const int32_t slot = slots[x / L];
                filt.push_back(FiltEntry{ev->div_buf[slot].as<float>() + ev->div_off[slot][x % L], e.list_off, e.n_blocks,
                                         (int32_t)sets[x].size()});
                most_blocks = std::max(most_blocks, e.n_blocks);
            }
            std::vector<double> filtered((size_t)list_total, 0.0);
            if (!filt.empty()) {
                upload(ev, ev->d_filt, filt.data(), filt.size() * sizeof(FiltEntry));
                upload(ev, ev->d_flags, in_set.data(), in_set.size() * sizeof(int32_t));
                hipLaunchKernelGGL(evict_filtered_diversity_kernel, dim3((unsigned)filt.size(), (unsigned)most_blocks),
                                   block, 0, ev->stream, ev->d_filt.as<FiltEntry>(), ev->d_flags.as<int32_t>(),
                                   ev->d_bscore.as<double>(), (int32_t)bsz);
                HIP_CHECK(hipGetLastError());
                HIP_CHECK(hipMemcpyAsync(filtered.data(), ev->d_bscore.p, filtered.size() * sizeof(double),
                                         hipMemcpyDeviceToHost, ev->stream));
                HIP_CHECK(hipStreamSynchronize(ev->stream));
            }
            pa::parallel_items(entries.size(), entries.size() / 64 + 1, [&](size_t x) {
                SelEntry& e = entries[x];
                if (e.n_blocks <= 0) return;
                std::set<size_t> keep;
                if (left[x] != 0) keep = calc.most_diverse_blocks(left[x], sets[x], filtered.data() + e.list_off);
                int32_t k = 0;
                for (size_t b : sets[x])
                    if (!keep.count(b)) lists[(size_t)e.list_off + k++] = (int32_t)b;
                PA_REQUIRE(k <= max_per_entry, PA_OUT_OF_BOUNDS, "more evicted blocks than the output holds");
                e.k = k;
            });
        } else {
            hipLaunchKernelGGL(evict_rank_kernel, grid, block, 0, ev->stream, ev->d_entries.as<SelEntry>(),
                               ev->d_bscore.as<double>(), ev->d_flags.as<int32_t>());
            hipLaunchKernelGGL(evict_list_kernel, grid, block, 0, ev->stream, ev->d_entries.as<SelEntry>(),
                               ev->d_flags.as<int32_t>(), ev->d_list.as<int32_t>());
            HIP_CHECK(hipGetLastError());
            HIP_CHECK(hipMemcpyAsync(lists.data(), ev->d_list.p, lists.size() * sizeof(int32_t), hipMemcpyDeviceToHost,
                                     ev->stream));
            HIP_CHECK(hipStreamSynchronize(ev->stream));
            lists_on_device = true;
            if (crush) {  // cache_eviction.cpp:367-398: some of the chosen blocks stay as representatives
                // Everything that walks tokens runs on the device (evict_crush_kernel); one distance per block comes
                // back.  Anchor points that do not depend on the scores are made here, in the order the reference
                // makes them (one per thinned entry, entries in call order: the random mode draws from the
                // sequence's generator), and go up with the entries.
                const int32_t mode = ev->cfg.kvcrush_anchor_point_mode;
                std::vector<CrushEntry> work;
                std::vector<size_t> work_entry;
                std::vector<uint8_t> anchors;
                int64_t dist_total = 0;
                for (size_t x = 0; x < entries.size(); ++x) {
                    const SelEntry& e = entries[x];
                    if (e.k <= 0 || (uint64_t)e.k < ev->cfg.kvcrush_budget) continue;
                    CrushEntry w{e.state_off, (int32_t)((size_t)e.n_blocks * bsz), (int32_t)dist_total, (int32_t)anchors.size(), 0};
                    if (mode != pa::ANCHOR_MEAN) {
                        std::vector<uint8_t> anchor;
                        PA_REQUIRE(ev->crush[slots[x / L]].anchor_point((size_t)w.n_tok, nullptr, anchor), PA_PARAMETER_MISMATCH,
                                   "Invalid anchor point type");
                        anchors.insert(anchors.end(), anchor.begin(), anchor.end());
                    }
                    work.push_back(w);
                    work_entry.push_back(x);
                    dist_total += e.n_blocks;
                    PA_REQUIRE(dist_total <= INT32_MAX, PA_OUT_OF_BOUNDS, "too many evictable blocks for one call");
                }
                if (!work.empty()) {
                    upload(ev, ev->d_gather_entries, work.data(), work.size() * sizeof(CrushEntry));
                    if (!anchors.empty()) upload(ev, ev->d_filt, anchors.data(), anchors.size());
                    // distances, then one flag per entry
                    const size_t back_ints = (size_t)dist_total + work.size();
                    ev->d_gather.reserve(back_ints * sizeof(int32_t));
                    ev->h_back.reserve(back_ints * sizeof(int32_t));
                    int32_t* d_dist = ev->d_gather.as<int32_t>();
                    hipLaunchKernelGGL(evict_crush_kernel, dim3((unsigned)work.size()), dim3(256), (size_t)bsz * sizeof(uint32_t),
                                       ev->stream, ev->d_gather_entries.as<CrushEntry>(), ev->scores,
                                       ev->d_filt.as<uint8_t>(), d_dist, d_dist + dist_total, (int32_t)bsz, mode);
                    HIP_CHECK(hipGetLastError());
                    HIP_CHECK(hipMemcpyAsync(ev->h_back.p, ev->d_gather.p, back_ints * sizeof(int32_t), hipMemcpyDeviceToHost,
                                             ev->stream));
                    HIP_CHECK(hipStreamSynchronize(ev->stream));
                    std::vector<int32_t> back(ev->h_back.as<int32_t>(), ev->h_back.as<int32_t>() + back_ints);
                    // entries whose top half is not settled by the scores alone: their token scores come back and the
                    // host walks them (same anchor point: the one made above, or the majority of the host's bits)
                    std::vector<GatherEntry> gather;
                    std::vector<size_t> gather_work;
                    int64_t packed = 0;
                    int32_t longest = 0;
                    for (size_t w = 0; w < work.size(); ++w) {
                        if (back[(size_t)dist_total + w] == 0) continue;
                        gather_work.push_back(w);
                        gather.push_back(GatherEntry{work[w].state_off, packed, work[w].n_tok, 0});
                        packed += work[w].n_tok;
                        longest = std::max(longest, work[w].n_tok);
                    }
                    if (!gather.empty()) {
                        upload(ev, ev->d_gather_entries, gather.data(), gather.size() * sizeof(GatherEntry));
                        ev->d_gather.reserve((size_t)packed * sizeof(double));
                        ev->h_back.reserve((size_t)packed * sizeof(double));
                        hipLaunchKernelGGL(evict_gather_kernel, dim3((unsigned)gather.size(), (unsigned)std::min(pa::ceil_div(longest, 256), 32)),
                                           dim3(256), 0, ev->stream, ev->d_gather_entries.as<GatherEntry>(), ev->scores,
                                           ev->d_gather.as<double>());
                        HIP_CHECK(hipGetLastError());
                        HIP_CHECK(hipMemcpyAsync(ev->h_back.p, ev->d_gather.p, (size_t)packed * sizeof(double), hipMemcpyDeviceToHost,
                                                 ev->stream));
                        HIP_CHECK(hipStreamSynchronize(ev->stream));
                        // (entries are independent and nothing below touches a selector's generator: host threads share them)
                        const double* tok_scores = ev->h_back.as<const double>();
                        auto walk = [&](size_t g) {
                            const size_t w = gather_work[g];
                            pa::KvCrushSelector& sel = ev->crush[slots[work_entry[w] / L]];
                            const size_t n_tok = (size_t)work[w].n_tok;
                            const std::vector<uint8_t> bits = sel.indicators(n_tok, tok_scores + gather[g].dst_off);
                            std::vector<uint8_t> anchor;
                            if (mode == pa::ANCHOR_MEAN) (void)sel.anchor_point(n_tok, bits.data(), anchor);
                            else anchor.assign(anchors.begin() + work[w].anchor_off, anchors.begin() + work[w].anchor_off + (long)bsz);
                            const std::vector<size_t> d = sel.hamming(n_tok, bits.data(), anchor.data());
                            for (size_t bidx = 0; bidx < d.size(); ++bidx) back[(size_t)work[w].dist_off + bidx] = (int32_t)d[bidx];
                        };
                        pa::parallel_items(gather.size(), (size_t)(packed / 65536 + 1), walk);
                    }
                    // the representatives: a sort of each entry's chosen blocks by distance, entries independent
                    std::atomic<bool> shortened{false};
                    pa::parallel_items(work.size(), work.size() / 64 + 1, [&](size_t w) {
                        SelEntry& e = entries[work_entry[w]];
                        int32_t* list = lists.data() + e.list_off;
                        const std::vector<size_t> chosen(list, list + e.k);
                        const std::vector<size_t> dist(back.begin() + work[w].dist_off, back.begin() + work[w].dist_off + e.n_blocks);
                        const std::vector<size_t> stay = ev->crush[slots[work_entry[w] / L]].representative(dist.data(), dist.size(), chosen);
                        std::vector<uint8_t> stays((size_t)e.n_blocks, 0);
                        for (size_t b : stay) stays[b] = 1;
                        int32_t k = 0;
                        for (size_t b : chosen)
                            if (!stays[b]) list[k++] = (int32_t)b;
                        if (k != e.k) shortened = true;
                        e.k = k;
                    });
                    if (shortened) lists_on_device = false;
                }
            }
        }
        if (!lists_on_device) {
            upload(ev, ev->d_entries, entries.data(), entries.size() * sizeof(SelEntry));
            upload(ev, ev->d_list, lists.data(), lists.size() * sizeof(int32_t));
        }
        compact(ev, entries);
        HIP_CHECK(hipStreamSynchronize(ev->stream));
        finish(lists.data(), false);
    });
}

int32_t pa_evictor_remove_scores(pa_evictor* ev, int32_t slot, int32_t layer, const int32_t* blocks, int32_t count) {
    if (!ev) return PA_INVALID_C_PARAM;
    return guarded(ev, [&] {
        check_slot(ev, slot);
        PA_REQUIRE(layer >= 0 && (uint64_t)layer < ev->L(), PA_OUT_OF_BOUNDS, "layer out of range");
        PA_REQUIRE(count >= 0 && (count == 0 || blocks), PA_INVALID_C_PARAM, "null argument");
        if (count == 0) return;
        uint64_t& len = ev->len[(uint64_t)slot * ev->L() + layer];
        for (int32_t i = 0; i < count; ++i) {
            PA_REQUIRE(blocks[i] >= 0 && (uint64_t)(blocks[i] + 1) * ev->cfg.block_size <= len, PA_OUT_OF_BOUNDS,
                       "block outside the tracked scores");
            PA_REQUIRE(i == 0 || blocks[i] > blocks[i - 1], PA_PARAMETER_MISMATCH, "blocks must be ascending");
        }
        HIP_CHECK(hipSetDevice(ev->cfg.device));
        std::vector<SelEntry> entries(1, SelEntry{ev->state_off(slot, layer), 0, (int32_t)len, 0, count, 0});
        upload(ev, ev->d_entries, entries.data(), sizeof(SelEntry));
        upload(ev, ev->d_list, blocks, (size_t)count * sizeof(int32_t));
        compact(ev, entries);
        HIP_CHECK(hipStreamSynchronize(ev->stream));
        len -= (uint64_t)count * ev->cfg.block_size;
        if (ev->rkv()) ev->clear_ring(slot, layer);  // cache_eviction.cpp:50
    });
}

int32_t pa_evictor_get_range(const pa_evictor* ev, int32_t slot, int32_t layer, uint64_t* begin, uint64_t* end) {
    if (!ev || !begin || !end) return PA_INVALID_C_PARAM;
    if (slot < 0 || (uint64_t)slot >= ev->cfg.max_sequences || layer < 0 || (uint64_t)layer >= ev->L())
        return PA_OUT_OF_BOUNDS;
    ev->range(slot, layer, begin, end);
    return PA_OK;
}

uint64_t pa_evictor_max_cache_size_after_eviction(const pa_evictor* ev) { return ev ? ev->max_after() : 0; }

int32_t pa_evictor_get_state(pa_evictor* ev, int32_t slot, int32_t layer, uint64_t* length, double* scores,
                             uint64_t* counters, uint64_t capacity) {
    if (!ev) return PA_INVALID_C_PARAM;
    return guarded(ev, [&] {
        check_slot(ev, slot);
        PA_REQUIRE(layer >= 0 && (uint64_t)layer < ev->L(), PA_OUT_OF_BOUNDS, "layer out of range");
        const uint64_t len = ev->len[(uint64_t)slot * ev->L() + layer];
        if (length) *length = len;
        const uint64_t n = std::min(len, capacity);
        if (n == 0 || (!scores && !counters)) return;
        HIP_CHECK(hipSetDevice(ev->cfg.device));
        HIP_CHECK(hipStreamSynchronize(ev->stream));
        const int64_t o = ev->state_off(slot, layer);
        if (scores) HIP_CHECK(hipMemcpy(scores, ev->scores + o, n * sizeof(double), hipMemcpyDeviceToHost));
        if (counters && ev->cfg.aggregation_mode == PA_AGG_NORM_SUM)
            HIP_CHECK(hipMemcpy(counters, ev->counters + o, n * sizeof(uint64_t), hipMemcpyDeviceToHost));
    });
}

int32_t pa_evictor_block_scores(pa_evictor* ev, int32_t slot, int32_t layer, double* out, uint64_t capacity,
                                uint64_t* count) {
    if (!ev) return PA_INVALID_C_PARAM;
    return guarded(ev, [&] {
        check_slot(ev, slot);
        PA_REQUIRE(layer >= 0 && (uint64_t)layer < ev->L() && out && count, PA_INVALID_C_PARAM, "bad argument");
        uint64_t rb, re;
        *count = 0;
        if (!ev->range(slot, layer, &rb, &re)) return;
        const uint64_t n = re - rb;
        HIP_CHECK(hipSetDevice(ev->cfg.device));
        std::vector<SelEntry> entries(1, SelEntry{ev->state_off(slot, layer), 0,
                                                  (int32_t)ev->len[(uint64_t)slot * ev->L() + layer], (int32_t)n, 0, 0});
        upload(ev, ev->d_entries, entries.data(), sizeof(SelEntry));
        ev->d_bscore.reserve(n * sizeof(double));
        hipLaunchKernelGGL(evict_block_score_kernel, dim3(1), dim3(256), 0, ev->stream, ev->d_entries.as<SelEntry>(),
                           ev->scores, ev->counters, ev->d_bscore.as<double>(), (int32_t)ev->cfg.block_size,
                           ev->cfg.aggregation_mode == PA_AGG_NORM_SUM ? 1 : 0);
        HIP_CHECK(hipGetLastError());
        HIP_CHECK(hipStreamSynchronize(ev->stream));
        *count = n;
        HIP_CHECK(hipMemcpy(out, ev->d_bscore.p, std::min(n, capacity) * sizeof(double), hipMemcpyDeviceToHost));
    });
}

}  // extern "C"
