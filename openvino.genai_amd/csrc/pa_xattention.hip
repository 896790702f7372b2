// Block-sparse prefill (XAttention): the importance estimate and the block selection that run before the matrix
// kernel for sequences whose `xattention_threshold` is above zero (model inputs `xattention_threshold.<L>`,
// `xattention_block_size`, `xattention_stride`, src/cpp/src/continuous_batching/model_runner.hpp:1623-1656).
//
// Positions are absolute.  Strided group i covers positions [i S, (i + 1) S); block I covers [I xb, (I + 1) xb).
//   1. logits:   a[h][i][j] = scale / S * sum_{s < S} q[i S + S-1-s] . k[j S + s]   for j <= i   (the antidiagonals
//                of the S x S tiles of Q K^T; tokens outside the chunk / beyond the context count as zero vectors)
//   2. per (head, I), one workgroup:
//        stats:  per strided group i of the block: maximum and denominator of the softmax over j = 0..i
//        sums:   B[h][I][J] = sum of the probabilities of the groups (i in I, j in J)
//        select: key blocks 0 and I, then the others in descending B (equal: lower J first) while the kept sum is
//                below threshold * sum_J B[h][I][J]  -> one bit per key block
//   3. lists:    per work item of the matrix kernel and kv head: which of its KV blocks any of its rows still needs
//
// Roofline: step 1 is dense MFMA work, 2 D / S flops per (query position, key position, head) -- 1 / (2 S) of the
// attention it prunes; the other steps touch a few hundred KB.
#include "pa_device.h"

#include <algorithm>

namespace pa {
namespace {

typedef _Float16 h8 __attribute__((ext_vector_type(8)));
typedef _Float16 h2 __attribute__((ext_vector_type(2)));
typedef __bf16 b8 __attribute__((ext_vector_type(8)));
typedef short s8v __attribute__((ext_vector_type(8)));
typedef float f4 __attribute__((ext_vector_type(4)));
typedef uint32_t u4v __attribute__((ext_vector_type(4)));

constexpr float LOG2E = 1.4426950408889634f;

template <int DT>
__device__ __forceinline__ f4 mma(const s8v& a, const s8v& b, const f4& c) {
    if (DT == DT_F16)
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(h8, a), __builtin_bit_cast(h8, b), c, 0, 0, 0);
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(b8, a), __builtin_bit_cast(b8, b), c, 0, 0, 0);
}

__device__ __forceinline__ uint32_t f16x2(float a, float b) {
    return __builtin_bit_cast(uint32_t, h2{(_Float16)a, (_Float16)b});
}

// ---- 1. strided logits ---------------------------------------------------------------------------------------
// A workgroup (four waves) = 32 strided query groups of up to four query heads that share a kv head x 64 strided
// key groups (XATT_KEY_TILE); wave w takes head w of the four: two 16-column tiles of queries (B operands) against
// four 16-row tiles of keys (A operands).  (With 128 key groups per workgroup -- half as many workgroups, 64
// accumulators -- the kernel took a quarter longer; stages of 128 channels instead of 64 changed nothing.)  The
// contraction runs over the S * D elements of a group in stages of (slot s, 64
// channels).  The stage's key rows (128 bytes each as 16-bit values) go global -> registers -> LDS once per
// workgroup and serve all four heads -- read straight from global memory by every wave, the same rows went through
// the L2 four times and that traffic, not the matrix pipe, set the pace.  u8 rows are dequantised on the way into
// LDS ((code - zero-point) * scale, rounded to f16), rows beyond the context are written as zeros.  Each wave's 32 query
// rows take the same way into an LDS buffer of the wave's own, eight lanes to a row's 128 bytes (loaded straight
// into operand layout -- sixteen rows per instruction, every lane in a cache line of its own -- the address unit set
// the pace).  Within a stage lane (n, g) supplies channels 16 g .. 16 g + 15 of row n as the k-slices of two matrix
// instructions (which channel sits in which k-slice is free as long as both operands agree).
template <int D, int DT, int QDT, bool U8>
__global__ __launch_bounds__(256, 2) void xatt_logits_kernel(XattArgs a) {
    static_assert(!U8 || DT == DT_F16, "u8 codes are multiplied as f16");
    constexpr int CROWB = U8 ? D + 8 : D * 2;
    constexpr int DP = D / 64;             // stages per slot
    constexpr int KST = 128;               // LDS bytes per key or query row of a stage; the row's 16-byte piece p sits at
                                           // p ^ ((row >> 1) & 7): stores (eight or four lanes to a row) and operand
                                           // reads (sixteen rows at one piece) both touch every bank once
    constexpr int KT = XATT_KEY_TILE;      // strided key groups per workgroup
    constexpr int NJ = KT / 16;
    constexpr int RPP = U8 ? 64 : 32;      // key rows one pass of the 256 threads covers
    constexpr int KCH = KT / RPP;          // 16-byte pieces of the cache a thread moves per stage
    __shared__ __align__(16) uint8_t kbuf[2][KT * KST];
    __shared__ __align__(16) uint8_t qbuf[2][4][32 * KST];   // per wave: its head's 32 query rows of a stage
    const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
    const int n = lane & 15, g = lane >> 4;
    const int Hq = a.sh.Hq, Hkv = a.sh.Hkv, G = a.G;
    const int nsub = (G + 3) >> 2;
    // Workgroup i runs on XCD i % 8, each with an L2 of its own.  The work is numbered (kv head, tile, set of four
    // heads) -- tiles in the order (sequence, query tile, key tile) -- and each XCD takes a contiguous eighth of that
    // numbering, so that the workgroups that read the same query rows (all key tiles of a query tile) and the same key
    // rows (both query tiles, all head sets) meet in one L2 instead of each fetching them over the fabric.
    const int total = gridDim.x, xcd = blockIdx.x & 7;
    const int work = xcd * (total >> 3) + min(xcd, total & 7) + (blockIdx.x >> 3);
    const int hkv = work / (a.ntiles * nsub);
    const int hg = (work % nsub) * 4 + wv;          // head within the group; waves beyond it repeat the last head
    const bool head_ok = hg < G;
    const int hq = hkv * G + min(hg, G - 1);
    const XattTile tl = a.tiles[(work / nsub) % a.ntiles];
    const XattSeq xs = a.seqs[tl.x];
    const int b = xs.b;
    const int t0 = a.st.subsequence_begins[b];
    const int q_len = a.st.subsequence_begins[b + 1] - t0;
    const int past = a.st.past_lens[b];
    const int kv_len = past + q_len;
    const int S = 1 << a.s_shift;
    const int32_t* table = a.block_indices + a.st.block_indices_begins[b];
    const int bs_shift = 31 - __builtin_clz(a.sh.bs);  // cache blocks of 32 tokens or more (a power of two)

    // this thread's share of a stage's key rows: rows kr0 + RPP * k, the piece `kpart` of each
    const int kr0 = U8 ? tid >> 2 : tid >> 3, kpart = U8 ? tid & 3 : tid & 7;
    int k_pos0[KCH];
    const uint8_t* k_blk[KCH];
#pragma unroll
    for (int k = 0; k < KCH; ++k) {
        k_pos0[k] = (KT * tl.jc + kr0 + RPP * k) << a.s_shift;
        const int pos = min(k_pos0[k], kv_len - 1);
        k_blk[k] = a.key_cache + ((long)table[pos >> bs_shift] * Hkv + hkv) * ((long)a.sh.bs * CROWB);
    }
    // this wave's query rows: a load covers eight rows, eight lanes to a row's 128 bytes; position of slot 0 (the
    // group's last token) of this lane's row in the first load, relative to the chunk
    const int qrow = lane >> 3, qpart = lane & 7;
    const int q_rel0 = ((xs.qs0 + 32 * tl.it + qrow) << a.s_shift) + S - 1 - past;
    struct KSet { u4v c[KCH]; uint2 hd[KCH]; };   // hd: u8 row headers
    struct QSet { u4v q[4]; };
    auto load_k = [&](KSet& ks, int u) __attribute__((always_inline)) {
        const int s = u / DP, ch = (u % DP) * 64;
#pragma unroll
        for (int k = 0; k < KCH; ++k) {
            const uint8_t* row = k_blk[k] + (min(k_pos0[k] + s, kv_len - 1) & (a.sh.bs - 1)) * CROWB;
            if (U8) {
                ks.c[k] = *reinterpret_cast<const u4v*>(row + 8 + ch + 16 * kpart);
                ks.hd[k] = *reinterpret_cast<const uint2*>(row);
            } else {
                ks.c[k] = *reinterpret_cast<const u4v*>(row + ch * 2 + 16 * kpart);
            }
        }
    };
    auto store_k = [&](const KSet& ks, int u) __attribute__((always_inline)) {
        const int s = u / DP;
        uint8_t* buf = kbuf[u & 1];
#pragma unroll
        for (int k = 0; k < KCH; ++k) {
            const bool ok = k_pos0[k] + s < kv_len;
            const int krow = kr0 + RPP * k, ksw = (krow >> 1) & 7;
            uint8_t* dst = buf + krow * KST;
            if (U8) {
                const float sc = ok ? __builtin_bit_cast(float, ks.hd[k].x) : 0.0f;
                const float nz = ok ? -__builtin_bit_cast(float, ks.hd[k].y) * sc : 0.0f;
                u4v v[2];
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const uint32_t w = ks.c[k][e];
                    v[e >> 1][2 * (e & 1)] = f16x2(fmaf((float)(w & 0xffu), sc, nz), fmaf((float)((w >> 8) & 0xffu), sc, nz));
                    v[e >> 1][2 * (e & 1) + 1] = f16x2(fmaf((float)((w >> 16) & 0xffu), sc, nz), fmaf((float)(w >> 24), sc, nz));
                }
                *reinterpret_cast<u4v*>(dst + 16 * ((2 * kpart) ^ ksw)) = v[0];
                *reinterpret_cast<u4v*>(dst + 16 * ((2 * kpart + 1) ^ ksw)) = v[1];
            } else {
                *reinterpret_cast<u4v*>(dst + 16 * (kpart ^ ksw)) = ok ? ks.c[k] : u4v{0u, 0u, 0u, 0u};
            }
        }
    };
    auto load_q = [&](QSet& qs, int u) __attribute__((always_inline)) {
        const int s = u / DP, ch = (u % DP) * 64 + 8 * qpart;
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            const int rel = q_rel0 + ((8 * c) << a.s_shift) - s;
            qs.q[c] = *reinterpret_cast<const u4v*>(a.query + ((long)(t0 + min(max(rel, 0), q_len - 1)) * Hq + hq) * D + ch);
        }
    };
    // rows outside the chunk go in as zeros; a bf16 query against f16 operands is converted here
    auto store_q = [&](const QSet& qs, int u) __attribute__((always_inline)) {
        const int s = u / DP;
        uint8_t* buf = qbuf[u & 1][wv];
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            const int rel = q_rel0 + ((8 * c) << a.s_shift) - s;
            u4v v = (rel >= 0 && rel < q_len) ? qs.q[c] : u4v{0u, 0u, 0u, 0u};
            if (QDT != DT) {
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    v[e] = f16x2(__builtin_bit_cast(float, v[e] << 16), __builtin_bit_cast(float, v[e] & 0xffff0000u));
            }
            const int row = 8 * c + qrow;
            *reinterpret_cast<u4v*>(buf + row * KST + 16 * (qpart ^ ((row >> 1) & 7))) = v;
        }
    };
    f4 acc[2][NJ];
#pragma unroll
    for (int mi = 0; mi < 2; ++mi)
#pragma unroll
        for (int nj = 0; nj < NJ; ++nj) acc[mi][nj] = f4{0.0f, 0.0f, 0.0f, 0.0f};
    auto compute = [&](int u) __attribute__((always_inline)) {
        const uint8_t* buf = kbuf[u & 1];
        const uint8_t* qb = qbuf[u & 1][wv];
#pragma unroll
        for (int kk = 0; kk < 2; ++kk) {
            s8v qop[2];
#pragma unroll
            for (int mi = 0; mi < 2; ++mi)
                qop[mi] = *reinterpret_cast<const s8v*>(qb + (16 * mi + n) * KST + 16 * ((2 * g + kk) ^ ((n >> 1) & 7)));
#pragma unroll
            for (int nj = 0; nj < NJ; ++nj) {
                const s8v kop = *reinterpret_cast<const s8v*>(buf + (16 * nj + n) * KST + 16 * ((2 * g + kk) ^ ((n >> 1) & 7)));
#pragma unroll
                for (int mi = 0; mi < 2; ++mi) acc[mi][nj] = mma<DT>(kop, qop[mi], acc[mi][nj]);
            }
        }
    };

    // stage u: its key and query rows were asked for in iteration u - 2 and written to LDS in iteration u - 1 (the
    // buffers (u + 1) & 1 were last read in iteration u - 1); the workgroups sharing a CU cover for each other.
    // (Four stages of loads in flight instead of one changed nothing: the pace is set by bytes, not by latency.)
    const int NU = S * DP;
    KSet k0, k1;
    QSet q0, q1;
    load_k(k0, 0);
    load_q(q0, 0);
    if (NU > 1) {
        load_k(k1, 1);
        load_q(q1, 1);
    }
    store_k(k0, 0);
    store_q(q0, 0);
    __syncthreads();
#define PA_XSTEP(KA, KB, QA, QB, U)                                      \
    {                                                                    \
        const int u = (U);                                               \
        if (u >= NU) break;                                              \
        if (u + 1 < NU) {                                                \
            store_k(KB, u + 1);                                          \
            store_q(QB, u + 1);                                          \
        }                                                                \
        if (u + 2 < NU) {                                                \
            load_k(KA, u + 2);                                           \
            load_q(QA, u + 2);                                           \
        }                                                                \
        compute(u);                                                      \
        __syncthreads();                                                 \
    }
    for (int i = 0;; i += 2) {
        PA_XSTEP(k0, k1, q0, q1, i)
        PA_XSTEP(k1, k0, q1, q0, i + 1)
    }
#undef PA_XSTEP

    // lane (n, g), register i of tile (mi, nj): query group 16 mi + n, key group 16 nj + 4 g + i
    if (!head_ok) return;
    const float scl = a.st.scale * LOG2E / (float)S;
    const int rows = (xs.nqs + 31) & ~31;
#pragma unroll
    for (int mi = 0; mi < 2; ++mi) {
        float* out = a.logits + xs.logit_off + ((long)hq * rows + 32 * tl.it + 16 * mi + n) * xs.ld + KT * tl.jc + 4 * g;
#pragma unroll
        for (int nj = 0; nj < NJ; ++nj) *reinterpret_cast<f4*>(out + 16 * nj) = acc[mi][nj] * scl;
    }
}

// ---- 2. statistics, block sums and selection of one (sequence, head, query block I) -------------------------
// One 256-thread workgroup.  (a) a wave per strided query group of the block: maximum and denominator of its
// softmax over j = 0 .. i; (b) a thread per key block J <= I: the probabilities of the block pair's groups, rows
// outer, columns inner; (c) the selection.  Sums are compared as fixed-point integers (value * 2^32, rounded to
// nearest), so that the kept sum does not depend on the order of the additions and the walk can be a parallel
// prefix sum: candidates J = 1 .. I - 1 are ranked by counting (value descending, equal values by ascending J), the
// candidate of rank k is taken iff the forced blocks plus the candidates of lower rank sum to less than
// threshold * total.  Dynamic LDS: see the launch.
__device__ __forceinline__ long long xatt_fixed(float v) { return __double2ll_rn((double)v * 4294967296.0); }

__global__ __launch_bounds__(256) void xatt_select_kernel(XattArgs a) {
    extern __shared__ __align__(16) uint8_t xsel_lds[];
    const XattSeq xs = a.seqs[blockIdx.z];
    const int hq = blockIdx.y, ib = blockIdx.x, tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
    if (ib >= xs.nqb) return;
    const int r_shift = a.xb_shift - a.s_shift, R = 1 << r_shift;
    long long* fx = reinterpret_cast<long long*>(xsel_lds);             // [max_nkb] fixed-point block sums
    long long* part = fx + a.max_nkb;                                   // [256] partial sums of the scan
    float* v = reinterpret_cast<float*>(part + 256);                    // [max_nkb]
    int32_t* order = reinterpret_cast<int32_t*>(v + a.max_nkb);         // [max_nkb]
    float2* stat = reinterpret_cast<float2*>(order + a.max_nkb);        // [R]
    uint32_t* bits = reinterpret_cast<uint32_t*>(stat + R);             // [words]
    const int I = xs.qb0 + ib;
    const int rows = (xs.nqs + 31) & ~31;
    const int i_lo = max(I << r_shift, xs.qs0), i_hi = min((I << r_shift) + R, xs.qs0 + xs.nqs);
    const float* logits = a.logits + xs.logit_off + (long)hq * rows * xs.ld;

    // (a) softmax statistics of the block's strided query groups: one pass, every lane keeps a running maximum and
    // the sum relative to it, the wave folds them
    for (int ig = i_lo + wv; ig < i_hi; ig += 4) {
        const float* row = logits + (long)(ig - xs.qs0) * xs.ld;
        float m = -INFINITY, l = 0.0f;
        // twenty values per lane and round, loaded before any is used (a round is a trip to memory that the next one
        // waits for: a row of up to 1280 strided keys takes one)
        for (int j0 = 4 * lane; j0 <= ig; j0 += 1280) {
            f4 xv[5];
#pragma unroll
            for (int c = 0; c < 5; ++c) xv[c] = *reinterpret_cast<const f4*>(row + min(j0 + 256 * c, xs.ld - 4));
            float x[20];
#pragma unroll
            for (int c = 0; c < 20; ++c) x[c] = j0 + 256 * (c >> 2) + (c & 3) <= ig ? xv[c >> 2][c & 3] : -INFINITY;
            float mx = x[0];
#pragma unroll
            for (int c = 1; c < 20; ++c) mx = fmaxf(mx, x[c]);
            const float mn = fmaxf(m, mx);  // finite: x[0] is a visible value
            float add = 0.0f;
#pragma unroll
            for (int c = 0; c < 20; ++c) add += __builtin_amdgcn_exp2f(x[c] - mn);
            l = l * __builtin_amdgcn_exp2f(m - mn) + add;
            m = mn;
        }
        const float M = wave_max(m);
        const float L = wave_sum(m == -INFINITY ? 0.0f : l * __builtin_amdgcn_exp2f(m - M));
        if (lane == 0) stat[ig - i_lo] = make_float2(M, 1.0f / L);
    }
    for (int w = tid; w < xs.words; w += 256) bits[w] = 0u;
    __syncthreads();
    // (b) block sums
    float* sums_out = a.sums + xs.sum_off + ((long)hq * xs.nqb + ib) * xs.nkb;
    for (int J = tid; J < xs.nkb; J += 256) {
        float total = 0.0f;
        if (J <= I && R == 8) {
            // the common shape (block 64, stride 8), unrolled so that the loads of all eight rows are in flight together;
            // rows the chunk does not have repeat a neighbour and count for nothing
            f4 x[8][2];
            float2 st[8];
#pragma unroll
            for (int r = 0; r < 8; ++r) {
                const int ig = min(max((I << 3) + r, i_lo), i_hi - 1);
                const float* rowp = logits + (long)(ig - xs.qs0) * xs.ld + (J << 3);
                x[r][0] = *reinterpret_cast<const f4*>(rowp);
                x[r][1] = *reinterpret_cast<const f4*>(rowp + 4);
                st[r] = stat[ig - i_lo];
            }
#pragma unroll
            for (int r = 0; r < 8; ++r) {
                const int ig = (I << 3) + r;
                float p = 0.0f;
#pragma unroll
                for (int c = 0; c < 8; ++c) p += (J << 3) + c <= ig ? __builtin_amdgcn_exp2f(x[r][c >> 2][c & 3] - st[r].x) : 0.0f;
                total = fmaf(p, ig >= i_lo && ig < i_hi ? st[r].y : 0.0f, total);
            }
        } else if (J <= I) {
            for (int ig = i_lo; ig < i_hi; ++ig) {
                const float* row = logits + (long)(ig - xs.qs0) * xs.ld;
                const float2 st = stat[ig - i_lo];
                const int j_hi = min((J << r_shift) + R, ig + 1);
                float p = 0.0f;
                for (int j = J << r_shift; j < j_hi; ++j) p += __builtin_amdgcn_exp2f(row[j] - st.x);
                total = fmaf(p, st.y, total);
            }
        }
        if (J <= I) {
            v[J] = total;
            fx[J] = xatt_fixed(total);
        }
        sums_out[J] = total;
    }
    __syncthreads();
    // (c) total and ranks
    const int ncand = max(I - 1, 0);  // candidates J = 1 .. I - 1
    long long mine = 0;
    for (int J = tid; J <= I; J += 256) mine += fx[J];
    for (int J = 1 + tid; J < I; J += 256) {
        const float my = v[J];
        int rank = 0;
        for (int o = 1; o < I; ++o) rank += (v[o] > my || (v[o] == my && o < J)) ? 1 : 0;
        order[rank] = J;
    }
    // the total: every wave adds its lanes' shares with lane swaps, the four wave sums meet in LDS (integers: the
    // same total in any order)
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) mine += __shfl_xor(mine, o, WAVE);
    if (lane == 0) part[wv] = mine;
    __syncthreads();  // (also: `order` is complete)
    const long long total_fx = part[0] + part[1] + part[2] + part[3];
    const long long forced = fx[0] + (I > 0 ? fx[I] : 0);
    const double required = (double)xs.threshold * (double)total_fx;
    // prefix sums over the ranked candidates: thread t owns ranks [t * per, (t + 1) * per); inclusive scan inside the
    // wave by lane shifts, the waves in front add their totals
    const int per = (ncand + 255) / 256;
    long long local = 0;
    for (int k = tid * per; k < min((tid + 1) * per, ncand); ++k) local += fx[order[k]];
    long long incl = local;
#pragma unroll
    for (int o = 1; o < WAVE; o <<= 1) {
        const long long up = __shfl_up(incl, o, WAVE);
        if (lane >= o) incl += up;
    }
    if (lane == WAVE - 1) part[4 + wv] = incl;
    __syncthreads();
    long long before = incl - local;  // the ranks in front of this thread's
    for (int w = 0; w < wv; ++w) before += part[4 + w];
    long long kept = forced + before;
    uint32_t* out = a.mask + xs.mask_off + ((long)hq * xs.nqb + ib) * xs.words;
    for (int k = tid * per; k < min((tid + 1) * per, ncand); ++k) {
        if (!((double)kept < required)) break;
        const int J = order[k];
        atomicOr(&bits[J >> 5], 1u << (J & 31));
        kept += fx[J];
    }
    if (tid == 0) {
        atomicOr(&bits[0], 1u);
        if (I > 0) atomicOr(&bits[I >> 5], 1u << (I & 31));
    }
    __syncthreads();
    for (int w = tid; w < xs.words; w += 256) out[w] = bits[w];
}

// ---- 3. the KV blocks a work item of the matrix kernel still needs ---------------------------------------
// One wave per (sparse item, kv head): lane t of pass p looks at KV block tb + 64 p + t, which is needed if any
// (query block, head of the group) among the item's rows kept the key block it lies in.  The needed ones are
// listed in ascending order behind their count.
__global__ __launch_bounds__(64) void xatt_item_keep_kernel(XattArgs a) {
    const int Hkv = a.sh.Hkv, lane = threadIdx.x;
    const int hkv = blockIdx.x % Hkv;
    const PrefillItem it = a.items[blockIdx.x / Hkv];
    const XattSeq xs = a.seqs[a.seq_of[it.b]];
    const int past = a.st.past_lens[it.b];
    const int qb_lo = (past + it.q0) >> a.xb_shift, qb_hi = (past + it.q0 + it.nq - 1) >> a.xb_shift;
    int32_t* list = a.item_tiles + (long)blockIdx.x * a.tiles_stride;
    int count = 0;
    for (int t0 = 0; t0 < it.te - it.tb; t0 += 64) {
        const int tile = it.tb + t0 + lane;
        // no early exit: the loads of all (query block, head) pairs should be in flight together
        const int J = min(tile, it.te - 1) >> (a.xb_shift - 5);
        uint32_t seen = 0u;
        for (int qb = qb_lo; qb <= qb_hi; ++qb) {
            const uint32_t* row = a.mask + xs.mask_off + ((long)hkv * a.G * xs.nqb + (qb - xs.qb0)) * xs.words + (J >> 5);
#pragma unroll 8
            for (int g = 0; g < a.G; ++g) seen |= row[(long)g * xs.nqb * xs.words];
        }
        const bool any = tile < it.te && ((seen >> (J & 31)) & 1u);
        const unsigned long long bal = __ballot(any);
        if (any) list[1 + count + __popcll(bal & ((1ull << lane) - 1ull))] = t0 + lane;
        count += __popcll(bal);
    }
    if (lane == 0) {
        list[0] = count;
        if (count == 0) list[1] = 0;  // the matrix kernel's clamped fetches still read one entry
    }
}

}  // namespace

hipError_t launch_xattention(hipStream_t s, const XattArgs& a, int q_dtype, int kv_dtype) {
    if (a.nseq == 0) return hipSuccess;
    const dim3 lgrid((unsigned)(a.ntiles * a.sh.Hkv * ceil_div(a.G, 4)));
#define PA_XLOGITS(DD, DT, Q, U8) \
    hipLaunchKernelGGL((xatt_logits_kernel<DD, DT, Q, U8>), lgrid, dim3(256), 0, s, a)
    const bool f16q = q_dtype == DT_F16;
    // (a stage is 64 channels of a slot: head sizes that are multiples of 64)
    if (a.sh.bs < 32 || a.sh.bs > 256 || (a.sh.bs & (a.sh.bs - 1)) || (a.sh.D != 64 && a.sh.D != 128 && a.sh.D != 256)) return hipErrorInvalidValue;
    if (kv_dtype == DT_U8) {
        if (a.sh.D == 64) { if (f16q) PA_XLOGITS(64, DT_F16, DT_F16, true); else PA_XLOGITS(64, DT_F16, DT_BF16, true); }
        else if (a.sh.D == 128) { if (f16q) PA_XLOGITS(128, DT_F16, DT_F16, true); else PA_XLOGITS(128, DT_F16, DT_BF16, true); }
        else { if (f16q) PA_XLOGITS(256, DT_F16, DT_F16, true); else PA_XLOGITS(256, DT_F16, DT_BF16, true); }
    } else if (kv_dtype == q_dtype) {
        if (a.sh.D == 64) { if (f16q) PA_XLOGITS(64, DT_F16, DT_F16, false); else PA_XLOGITS(64, DT_BF16, DT_BF16, false); }
        else if (a.sh.D == 128) { if (f16q) PA_XLOGITS(128, DT_F16, DT_F16, false); else PA_XLOGITS(128, DT_BF16, DT_BF16, false); }
        else { if (f16q) PA_XLOGITS(256, DT_F16, DT_F16, false); else PA_XLOGITS(256, DT_BF16, DT_BF16, false); }
    } else {
        return hipErrorInvalidValue;
    }
#undef PA_XLOGITS
    const int R = 1 << (a.xb_shift - a.s_shift);
    const size_t lds = (size_t)a.max_nkb * 16 + 256 * 8 + (size_t)R * 8 + (size_t)ceil_div(a.max_nkb, 32) * 4;
    hipLaunchKernelGGL(xatt_select_kernel, dim3((unsigned)a.max_nqb, (unsigned)a.sh.Hq, (unsigned)a.nseq), dim3(256), lds,
                       s, a);
    if (a.n_items > 0)
        hipLaunchKernelGGL(xatt_item_keep_kernel, dim3((unsigned)(a.n_items * a.sh.Hkv)), dim3(64), 0, s, a);
    return hipGetLastError();
}

}  // namespace pa
