// Block diversity of the evictable area for ADAPTIVE_RKV eviction, on the gfx950 matrix cores.
//
// Per sequence, with K the key rows of its `ev` evictable tokens (positions start .. start + ev of the paged cache)
// and one kv head at a time:
//   k^ = k / sqrt(|k|^2 + eps)                      unit rows
//   S  = K^ K^T, diagonal set to 0                  cosine similarity of every token pair
//   S[r][c] = 0 where S[r][c] < mean_c S[r][c]      entries below their row's mean are dropped
//   A  = mean over kv heads of S
//   out[rb][c] = - sum over the 32 rows r of block rb of A[r][c]         [ev / 32, ev] values per sequence
//
// Four kernels.  The first three are O(ev * D) preparation, sixteen lanes per token row:
//   rkv_stats_colsum_kernel : per (head, token) the factor that normalises the row, and for u8 rows the zero-point
//                       and the sum of the codes; the sum of the unit rows over chunks of 256 tokens (fixed order);
//   rkv_total_kernel  : the chunks' sums added up in chunk order;
//   rkv_mean_kernel   : row mean of S with its diagonal zeroed = (k^_r . sum_c k^_c - k^_r . k^_r) / ev, which
//                       costs a dot product per row instead of a pass over the similarity matrix.
// rkv_diversity_kernel is the O(ev^2 * D) part: a wave owns 32-row blocks and 64 columns, holds the columns of one kv
// head as MFMA operands (lane (n, g): token 16 t + n, channels 32 s + 8 g .. + 7) and reads the rows, which its
// workgroup shares, from LDS; it forms the 32 x 64 tiles of raw dot products with v_mfma_f32_16x16x32_{f16,bf16},
// scales / masks them in registers and adds the rows up; heads accumulate in registers, so every output value is
// written once, by one lane, in a fixed order (no atomics).
// u8 caches: the codes are multiplied exactly as f16 subnormals (code * 2^-24, products summed in f32 without
// rounding: at most 128 * 255^2 < 2^24), and scale / zero-point enter on the accumulator:
//   k_r . k_c = sc_r sc_c (sum(c_r c_c) - zp_c sum(c_r) - zp_r sum(c_c) + D zp_r zp_c).
//
// Roofline: dense MFMA (2 * D flops per token pair and head); the operand rows come from L2 (every row is read
// by ev / 256 workgroups as a row and ev / 128 or ev / 32 waves as a column).
#include "pa_device.h"

namespace pa {
namespace {

typedef _Float16 h8 __attribute__((ext_vector_type(8)));
typedef __bf16 b8 __attribute__((ext_vector_type(8)));
typedef short s8v __attribute__((ext_vector_type(8)));
typedef float f4 __attribute__((ext_vector_type(4)));
typedef uint32_t u4v __attribute__((ext_vector_type(4)));
typedef uint32_t u2v __attribute__((ext_vector_type(2)));

constexpr float NORM_EPS = 1e-12f;
constexpr int CHUNK = 256;  // tokens per partial column sum

template <int DT>
__device__ __forceinline__ f4 mma(const s8v& a, const s8v& b, const f4& c) {
    if (DT == DT_F16)
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(h8, a), __builtin_bit_cast(h8, b), c, 0, 0, 0);
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(b8, a), __builtin_bit_cast(b8, b), c, 0, 0, 0);
}

// The preparation kernels give a token row to 16 lanes, D / 16 consecutive channels each (8 or 16 bytes per lane at
// D = 128), four rows per wave and load.  The lane's channels as floats (u8: dequantised), and for u8 the codes.
template <int D, int KVDT>
__device__ __forceinline__ void lane_channels(const uint8_t* row, int l16, float (&x)[D / 16], float (&code)[D / 16]) {
    constexpr int E = D / 16;
    static_assert(E == 4 || E == 6 || E == 8 || E == 16, "head size 64, 96, 128 or 256");
    if (KVDT == DT_U8) {
        const float2 hd = *reinterpret_cast<const float2*>(row);
        uint32_t w[(E + 3) / 4];
        const uint8_t* p = row + 8 + E * l16;
        if constexpr (E == 16) {  // (rows start on 8-byte boundaries)
            const u2v v0 = *reinterpret_cast<const u2v*>(p), v1 = *reinterpret_cast<const u2v*>(p + 8);
            w[0] = v0[0], w[1] = v0[1], w[2] = v1[0], w[3] = v1[1];
        } else if constexpr (E == 8) {
            const u2v v = *reinterpret_cast<const u2v*>(p);
            w[0] = v[0];
            w[1] = v[1];
        } else if constexpr (E == 6) {  // (six bytes on a 2-byte boundary)
            const uint16_t* h = reinterpret_cast<const uint16_t*>(p);
            w[0] = (uint32_t)h[0] | ((uint32_t)h[1] << 16);
            w[1] = h[2];
        } else {
            w[0] = *reinterpret_cast<const uint32_t*>(p);
        }
#pragma unroll
        for (int e = 0; e < E; ++e) {
            code[e] = (float)((w[e / 4] >> (8 * (e % 4))) & 0xffu);
            x[e] = (code[e] - hd.y) * hd.x;
        }
    } else {
        uint32_t w[E / 2];
        const uint8_t* p = row + 2 * E * l16;
        if constexpr (E % 8 == 0) {
#pragma unroll
            for (int j = 0; j < E / 8; ++j) {
                const u4v v = *reinterpret_cast<const u4v*>(p + 16 * j);
#pragma unroll
                for (int i = 0; i < 4; ++i) w[4 * j + i] = v[i];
            }
        } else if constexpr (E == 6) {  // (twelve bytes on a 4-byte boundary)
#pragma unroll
            for (int i = 0; i < 3; ++i) w[i] = reinterpret_cast<const uint32_t*>(p)[i];
        } else {
            const u2v v = *reinterpret_cast<const u2v*>(p);
            w[0] = v[0];
            w[1] = v[1];
        }
#pragma unroll
        for (int e = 0; e < E; ++e) {
            code[e] = 0.0f;
            x[e] = load16<KVDT>((uint16_t)(w[e / 2] >> (16 * (e % 2))));
        }
    }
}

// One pass over the area's rows, a workgroup per (sequence, head, chunk of 256 tokens):
//   stats[h][token] = { factor that turns the raw dot product of two rows into their cosine (1 / |k|, times the
//                       row's scale for u8), zero-point, sum of codes, k^ . k^ }
//   colsum[seq][h][chunk][d] = sum of k^[d] over the chunk's tokens: each of the workgroup's sixteen 16-lane groups
//                       adds tokens group, group + 16, ... in order, the groups' sums are added in group order.
template <int D, int KVDT>
__global__ __launch_bounds__(256) void rkv_stats_colsum_kernel(RkvDivArgs a) {
    constexpr int E = D / 16;
    __shared__ float red[16][D];
    const RkvDivSeq q = a.seqs[blockIdx.z];
    const int h = blockIdx.y;
    const int base = blockIdx.x * CHUNK;
    if (base >= q.ev) return;
    const int l16 = threadIdx.x & 15, grp = threadIdx.x >> 4;
    float acc[E];
#pragma unroll
    for (int e = 0; e < E; ++e) acc[e] = 0.0f;
    constexpr int CROWB = KVDT == DT_U8 ? D + 8 : D * 2;
    const int32_t* table = a.block_indices + q.table_off + q.first_block;
    const int last_blk = q.ev / 32 - 1;
#pragma unroll 4
    for (int i = 0; i < CHUNK / 16; ++i) {
        const int j = base + grp + 16 * i;
        const bool live = j < q.ev;
        // rows beyond the area repeat a row of its last block: the loads are unconditional, so that an unrolled round's
        // loads are in flight together; such rows add zeros and write nothing.  (The block is the same for the whole
        // workgroup: base is a multiple of 32 and grp below 16, so its id is read once, by the scalar unit.)
        const int32_t phys = table[min(base / 32 + (i >> 1), last_blk)];
        const uint8_t* row = a.key_cache + (((long)phys * a.Hkv + h) * 32 + (grp + 16 * (i & 1))) * CROWB;
        float x[E], code[E];
        lane_channels<D, KVDT>(row, l16, x, code);
        float sq = 0.0f, cs = 0.0f;
#pragma unroll
        for (int e = 0; e < E; ++e) {
            sq = fmaf(x[e], x[e], sq);
            cs += code[e];
        }
        sq = row16_sum(sq);
        cs = row16_sum(cs);  // integers below 2^24: exact in any order
        const float inv = 1.0f / sqrtf(sq + NORM_EPS);
#pragma unroll
        for (int e = 0; e < E; ++e) acc[e] += live ? x[e] * inv : 0.0f;
        if (l16 == 0 && live) {
            float sc = 1.0f, zp = 0.0f;
            if (KVDT == DT_U8) {
                const float2 hd = *reinterpret_cast<const float2*>(row);
                sc = hd.x;
                zp = hd.y;
            }
            a.stats[(long)h * a.total_tok + q.tok_off + j] = make_float4(sc * inv, zp, cs, sq * inv * inv);
        }
    }
#pragma unroll
    for (int e = 0; e < E; ++e) red[grp][l16 * E + e] = acc[e];
    __syncthreads();
    if (threadIdx.x < D) {
        float s = red[0][threadIdx.x];
#pragma unroll
        for (int k = 1; k < 16; ++k) s += red[k][threadIdx.x];
        a.colsum[(((long)blockIdx.z * a.Hkv + h) * (a.chunks_max + 1) + 1 + blockIdx.x) * D + threadIdx.x] = s;
    }
}

// colsum[seq][h][0][d] = sum over the chunks, in chunk order.
template <int D>
__global__ __launch_bounds__(D) void rkv_total_kernel(RkvDivArgs a) {
    const RkvDivSeq q = a.seqs[blockIdx.y];
    const int chunks = (q.ev + CHUNK - 1) / CHUNK;
    float* cs = a.colsum + ((long)blockIdx.y * a.Hkv + blockIdx.x) * (a.chunks_max + 1) * D;
    float s = 0.0f;
#pragma unroll 4
    for (int c = 0; c < chunks; ++c) s += cs[(long)(1 + c) * D + threadIdx.x];
    cs[threadIdx.x] = s;
}

// mean[h][token] = (k^_r . sum over the area's tokens of k^ - k^_r . k^_r) / ev, divided by the row's factor; a
// workgroup takes 128 tokens, each 16-lane group eight of them, whose loads go out together.
template <int D, int KVDT>
__global__ __launch_bounds__(256) void rkv_mean_kernel(RkvDivArgs a) {
    constexpr int E = D / 16;
    constexpr int TPG = 8;
    const RkvDivSeq q = a.seqs[blockIdx.z];
    const int h = blockIdx.y;
    const int l16 = threadIdx.x & 15, grp = threadIdx.x >> 4;
    const int j0 = blockIdx.x * (16 * TPG) + grp;   // tokens j0, j0 + 16, ..
    if (blockIdx.x * (16 * TPG) >= q.ev) return;
    const float* tot = a.colsum + ((long)blockIdx.z * a.Hkv + h) * (a.chunks_max + 1) * D;
    float s[E];
#pragma unroll
    for (int e = 0; e < E; ++e) s[e] = tot[l16 * E + e];
    constexpr int CROWB = KVDT == DT_U8 ? D + 8 : D * 2;
    const int32_t* table = a.block_indices + q.table_off + q.first_block;
    const int last_blk = q.ev / 32 - 1;
    float dot[TPG], self[TPG], fac[TPG];
#pragma unroll
    for (int t = 0; t < TPG; ++t) {
        // (tokens beyond the area: a row of its last block, nothing is written for them; the block is the same for the
        // whole workgroup, so its id is read by the scalar unit)
        const int blk = min(blockIdx.x * (TPG / 2) + (t >> 1), last_blk);
        const int j = blk * 32 + grp + 16 * (t & 1);
        const float4 st = a.stats[(long)h * a.total_tok + q.tok_off + j];
        const uint8_t* row = a.key_cache + (((long)table[blk] * a.Hkv + h) * 32 + (grp + 16 * (t & 1))) * CROWB;
        float x[E], code[E];
        lane_channels<D, KVDT>(row, l16, x, code);
        float d = 0.0f;
#pragma unroll
        for (int e = 0; e < E; ++e) d = fmaf(KVDT == DT_U8 ? (code[e] - st.y) * st.x : x[e] * st.x, s[e], d);
        dot[t] = d;
        self[t] = st.w;
        fac[t] = st.x;
    }
#pragma unroll
    for (int t = 0; t < TPG; ++t) dot[t] = row16_sum(dot[t]);
    if (l16 == 0) {
#pragma unroll
        for (int t = 0; t < TPG; ++t)
            if (j0 + 16 * t < q.ev)  // stored over the row's factor: what the raw product times the column's factor is held against
                a.mean[(long)h * a.total_tok + q.tok_off + j0 + 16 * t] = (dot[t] - self[t]) / (float)q.ev / fac[t];
    }
}

// DT: MFMA operand type (f16 for f16 and u8 caches, bf16 for bf16 caches).  RB: 32-row blocks per workgroup.
// A workgroup owns RB row blocks and 256 columns, 64 to a wave.  Per kv head the rows of its RB blocks and their
// per-row terms go global -> registers -> LDS once (coalesced: a row block of one head is contiguous in the cache) and
// serve all four waves; the wave's 64 columns stay in registers for the head.  (With every wave loading rows and
// per-row terms straight into operand layout, 9 KB per 16 matrix instructions came back through the vector memory
// path, which then set the pace: 15 % of the matrix peak.)  The next head's rows are asked for before the current
// head's arithmetic and written to LDS behind it.
// LDS rows hold operands: 2 D bytes (u8 codes widened to 16 bits on the way in, once per workgroup instead of once
// per wave and use) + 16 bytes of padding (the 16-byte operand reads of sixteen rows touch every bank).
template <int D, bool U8, int RB>
struct RkvTile {
    static constexpr int CROWB = U8 ? D + 8 : D * 2;
    static constexpr int ROWS = RB * 32;
    static constexpr int LROW = D * 2 + 16;
    static constexpr int BLKB = 32 * LROW;                 // LDS bytes of one row block
    static constexpr int PIECES = 32 * D / 8;              // pieces (eight channels: 8 bytes of codes, or 16 bytes) of a (block, head)
    static constexpr int PPT = (PIECES + 255) / 256;       // pieces per thread and row block
    static constexpr int OPB = RB * BLKB;
    static constexpr int LDSB = OPB + ROWS * 16;           // operands | per-row terms {factor, zero-point, code sum, threshold}
};

template <int D, int DT, bool U8, int RB>
__global__ __launch_bounds__(256) void rkv_diversity_kernel(RkvDivArgs a) {
    using T = RkvTile<D, U8, RB>;
    constexpr int KS = D / 32;
    constexpr int CROWB = T::CROWB;
    constexpr float CODE_UNIT2 = 281474976710656.0f;  // 2^48: both operands are code * 2^-24
    __shared__ __align__(16) uint8_t lds[T::LDSB];
    const RkvDivSeq q = a.seqs[blockIdx.z];
    const int rb0 = blockIdx.y * RB;
    const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
    if (rb0 * 32 >= q.ev || blockIdx.x * 256 >= q.ev) return;  // (the whole workgroup)
    const int col0 = (blockIdx.x * 4 + wv) * 64;
    const bool wave_live = col0 < q.ev;  // a wave beyond the area still moves rows and meets the barriers
    const int n = lane & 15, g = lane >> 4;
    const int last_rb = q.ev / 32 - 1;

    // physical blocks of the wave's column tokens and of the workgroup's row blocks, looked up once for all heads
    const int32_t* table = a.block_indices + q.table_off + q.first_block;
    long col_off[4], blk_off[RB];
#pragma unroll
    for (int c = 0; c < 4; ++c) {
        const int j = min(col0 + 16 * c + n, q.ev - 1);  // columns beyond the area repeat its last token
        col_off[c] = ((long)table[j >> 5] * a.Hkv * 32 + (j & 31)) * CROWB;
    }
#pragma unroll
    for (int k = 0; k < RB; ++k)  // row blocks beyond the area repeat its last one; their sums are never written
        blk_off[k] = (long)table[min(rb0 + k, last_rb)] * a.Hkv * 32 * CROWB;

    auto col_operand = [&](int h, long off, s8v (&reg)[KS]) __attribute__((always_inline)) {
        const uint8_t* row = a.key_cache + off + (long)h * 32 * CROWB;
#pragma unroll
        for (int s = 0; s < KS; ++s) {
            u4v v;
            if (U8) {
                const u2v cd = *reinterpret_cast<const u2v*>(row + 8 + 32 * s + 8 * g);
                v = u4v{__builtin_amdgcn_perm(0u, cd[0], 0x0c010c00u), __builtin_amdgcn_perm(0u, cd[0], 0x0c030c02u),
                        __builtin_amdgcn_perm(0u, cd[1], 0x0c010c00u), __builtin_amdgcn_perm(0u, cd[1], 0x0c030c02u)};
            } else {
                v = *reinterpret_cast<const u4v*>(row + (32 * s + 8 * g) * 2);
            }
            reg[s] = __builtin_bit_cast(s8v, v);
        }
    };
    // a head's rows and per-row terms on their way to LDS: thread tid moves pieces tid, tid + 256, .. of every row
    // block and the terms of row tid
    constexpr int PPR = D / 8;  // pieces per row
    struct Staged {
        u4v piece[RB][T::PPT];  // (u8: the first two words)
        float4 terms;
    };
    auto fetch = [&](Staged& sg, int h) __attribute__((always_inline)) {
#pragma unroll
        for (int k = 0; k < RB; ++k) {
            const uint8_t* src = a.key_cache + blk_off[k] + (long)h * 32 * CROWB;
#pragma unroll
            for (int i = 0; i < T::PPT; ++i) {
                const int p = min(tid + 256 * i, T::PIECES - 1);
                if (U8) {
                    const u2v cd = *reinterpret_cast<const u2v*>(src + (p / PPR) * CROWB + 8 + 8 * (p % PPR));
                    sg.piece[k][i] = u4v{cd[0], cd[1], 0u, 0u};
                } else {
                    sg.piece[k][i] = *reinterpret_cast<const u4v*>(src + 16 * p);
                }
            }
        }
        if (tid < T::ROWS) {
            const long r = (long)h * a.total_tok + q.tok_off + min(rb0 + (tid >> 5), last_rb) * 32 + (tid & 31);
            const float4 st = a.stats[r];
            sg.terms = make_float4(st.x, st.y, st.z * (1.0f / CODE_UNIT2), a.mean[r]);
        }
    };
    auto put = [&](const Staged& sg) __attribute__((always_inline)) {
#pragma unroll
        for (int k = 0; k < RB; ++k)
#pragma unroll
            for (int i = 0; i < T::PPT; ++i) {
                const int p = tid + 256 * i;
                if (p < T::PIECES) {
                    u4v v = sg.piece[k][i];
                    if (U8)  // code bytes to 16-bit words: code * 2^-24 as f16
                        v = u4v{__builtin_amdgcn_perm(0u, v[0], 0x0c010c00u), __builtin_amdgcn_perm(0u, v[0], 0x0c030c02u),
                                __builtin_amdgcn_perm(0u, v[1], 0x0c010c00u), __builtin_amdgcn_perm(0u, v[1], 0x0c030c02u)};
                    *reinterpret_cast<u4v*>(lds + k * T::BLKB + (p / PPR) * T::LROW + 16 * (p % PPR)) = v;
                }
            }
        if (tid < T::ROWS) *reinterpret_cast<float4*>(lds + T::OPB + 16 * tid) = sg.terms;
    };

    // Per element the vector unit does little: with raw = the accumulator, a_r / a_c the rows' factors and m_r the
    // row mean,
    //   v = raw' * a_c,  kept where v >= m_r / a_r,  column sum += v * a_r
    // and for u8 rows raw' = raw - zp_c * sum(c_r) - zp_r * (sum(c_c) - D zp_c), the powers of two of the code
    // unit folded into the per-row and per-column terms.  The diagonal is only looked for in the one 16 x 16 tile
    // per row tile that holds it.
    float colacc[RB][4];
#pragma unroll
    for (int k = 0; k < RB; ++k)
#pragma unroll
        for (int c = 0; c < 4; ++c) colacc[k][c] = 0.0f;
    Staged sg;
    fetch(sg, 0);
    put(sg);
    __syncthreads();
    for (int h = 0; h < a.Hkv; ++h) {
        const long sbase = (long)h * a.total_tok + q.tok_off;
        if (h + 1 < a.Hkv) fetch(sg, h + 1);
        s8v breg[4][KS];
        // (no branch around the loads of columns beyond the area; they are never written)
#pragma unroll
        for (int c = 0; c < 4; ++c) col_operand(h, col_off[c], breg[c]);
        float c_fac[4], c_zp[4], c_w[4];
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            const float4 st = a.stats[sbase + min(col0 + 16 * c + n, q.ev - 1)];
            c_fac[c] = U8 ? st.x * CODE_UNIT2 : st.x;
            c_zp[c] = st.y;
            c_w[c] = (st.z - (float)D * st.y) * (1.0f / CODE_UNIT2);
        }
        if (wave_live) {
#pragma unroll
            for (int k = 0; k < RB; ++k) {
                const int rb = min(rb0 + k, last_rb);
#pragma unroll
                for (int t = 0; t < 2; ++t) {
                    s8v areg[KS];
                    const uint8_t* row = lds + k * T::BLKB + (16 * t + n) * T::LROW;
#pragma unroll
                    for (int s = 0; s < KS; ++s)
                        areg[s] = __builtin_bit_cast(s8v, *reinterpret_cast<const u4v*>(row + (32 * s + 8 * g) * 2));
                    float4 rt[4];  // {factor, zero-point, code sum, threshold} of rows 16 t + 4 g + i
#pragma unroll
                    for (int i = 0; i < 4; ++i)
                        rt[i] = *reinterpret_cast<const float4*>(lds + T::OPB + 16 * (32 * k + 16 * t + 4 * g + i));
#pragma unroll
                    for (int c = 0; c < 4; ++c) {
                        f4 acc = f4{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
                        for (int s = 0; s < KS; ++s) acc = mma<DT>(areg[s], breg[c][s], acc);
                        float v[4];
#pragma unroll
                        for (int i = 0; i < 4; ++i) {
                            float raw = acc[i];
                            if (U8) raw = fmaf(-rt[i].y, c_w[c], fmaf(-c_zp[c], rt[i].z, raw));
                            v[i] = raw * c_fac[c];
                        }
                        if (rb * 32 + 16 * t == col0 + 16 * c) {  // (uniform) the tile that holds the diagonal
#pragma unroll
                            for (int i = 0; i < 4; ++i)
                                if (4 * g + i == n) v[i] = 0.0f;
                        }
#pragma unroll
                        for (int i = 0; i < 4; ++i) colacc[k][c] = fmaf(v[i] < rt[i].w ? 0.0f : v[i], rt[i].x, colacc[k][c]);
                    }
                }
            }
        }
        __syncthreads();  // every wave is done with this head's rows
        if (h + 1 < a.Hkv) put(sg);
        __syncthreads();
    }
    if (!wave_live) return;
    const float inv_h = 1.0f / (float)a.Hkv;
#pragma unroll
    for (int k = 0; k < RB; ++k) {
        float* out = a.out + q.out_off + (long)(rb0 + k) * q.ev;
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            float v = colacc[k][c];
            v += __shfl_xor(v, 16, WAVE);
            v += __shfl_xor(v, 32, WAVE);
            const int col = col0 + 16 * c + n;
            if (g == 0 && col < q.ev && rb0 + k <= last_rb) out[col] = -(v * inv_h);
        }
    }
}

template <int D, int KVDT>
hipError_t launch_typed(hipStream_t s, const RkvDivArgs& a, int nseq, int ev_max) {
    constexpr int DT = KVDT == DT_BF16 ? DT_BF16 : DT_F16;
    const dim3 block(256);
    const int chunks = ceil_div(ev_max, CHUNK);
    hipLaunchKernelGGL((rkv_stats_colsum_kernel<D, KVDT>), dim3((unsigned)chunks, (unsigned)a.Hkv, (unsigned)nseq), block, 0,
                       s, a);
    hipLaunchKernelGGL((rkv_total_kernel<D>), dim3((unsigned)a.Hkv, (unsigned)nseq), dim3(D), 0, s, a);
    hipLaunchKernelGGL((rkv_mean_kernel<D, KVDT>), dim3((unsigned)ceil_div(ev_max, 128), (unsigned)a.Hkv, (unsigned)nseq),
                       block, 0, s, a);
    // four row blocks per wave once that still leaves a few thousand waves
    const long waves4 = (long)nseq * ceil_div(ev_max, 128) * ceil_div(ev_max, 64);
    // (head size 256: the columns' operands alone are 128 registers, four row blocks would spill)
    bool four = false;
    if constexpr (D <= 128) {
        four = waves4 >= 4096;
        if (four)
            hipLaunchKernelGGL((rkv_diversity_kernel<D, DT, KVDT == DT_U8, 4>),
                               dim3((unsigned)ceil_div(ev_max, 256), (unsigned)ceil_div(ev_max, 128), (unsigned)nseq), block, 0, s, a);
    }
    if (!four)
        hipLaunchKernelGGL((rkv_diversity_kernel<D, DT, KVDT == DT_U8, 1>),
                           dim3((unsigned)ceil_div(ev_max, 256), (unsigned)(ev_max / 32), (unsigned)nseq), block, 0, s, a);
    return hipGetLastError();
}

}  // namespace

int rkv_diversity_chunks(int ev_max) { return ceil_div(ev_max, CHUNK); }

hipError_t launch_rkv_diversity(hipStream_t s, const RkvDivArgs& a, int kv_dtype, int D, int bs, int nseq, int ev_max) {
    if (nseq == 0 || ev_max == 0) return hipSuccess;
    if (bs != 32 || ev_max % 32) return hipErrorInvalidValue;
#define PA_DIV(D_)                                                                        \
    if (D == D_) {                                                                        \
        if (kv_dtype == DT_U8) return launch_typed<D_, DT_U8>(s, a, nseq, ev_max);        \
        if (kv_dtype == DT_F16) return launch_typed<D_, DT_F16>(s, a, nseq, ev_max);      \
        if (kv_dtype == DT_BF16) return launch_typed<D_, DT_BF16>(s, a, nseq, ev_max);    \
    }
    PA_DIV(128)
    PA_DIV(64)
    PA_DIV(96)
    PA_DIV(256)
#undef PA_DIV
    return hipErrorInvalidValue;
}

}  // namespace pa
