// Decode (q_len = 1) PagedAttention over a u8 KV cache: a bandwidth-bound split-K flash-decoding
// kernel for gfx950.
//
// Work item = (sequence, kv head, split): one 256-thread workgroup, four waves taking the split's
// 32-token KV blocks round-robin.  Per block and wave:
//   * the K block (32 rows x (8 B header + D codes), contiguous in the cache) and the V block are
//     fetched with fully coalesced 16-byte loads, one block ahead of the arithmetic, and staged
//     through a wave-private LDS slot to re-shape them into MFMA operand layout;
//   * u8 codes become fp16 operands in registers with one byte-permute per code pair: the
//     zero-extended byte IS the fp16 subnormal code * 2^-24, which the gfx950 matrix cores take
//     without flushing; scale / zero-point are applied to the 16x16 accumulator tiles instead
//     of to the D-wide rows:
//         logit  = scale * sc_k * (q . codes - zp_k * sum(q))
//         out    = sum_t p_t sc_v (codes_t - zp_v) = sum_t w_t codes_t - sum_t w_t zp_v
//   * QK and PV run on v_mfma_f32_16x16x32_f16 with the GQA group (<= 16 query heads sharing the
//     kv head) as the N dimension, so every cache byte is read once for the whole group;
//   * softmax is online, in the log2 domain, per wave; waves and splits merge at the end.
// Scores: the un-normalised probabilities of a workgroup's positions stay in LDS (fp16, relative
// to the running maximum, which is snapshotted per block); once the final maximum and denominator
// are known they are normalised, summed over the group's heads and written out.
//
// Roofline: HBM.  Algorithmic bytes per (sequence, kv head, position): 2 * (D + 8).
#include <type_traits>

#include "pa_device.h"

namespace pa {
namespace {

typedef _Float16 h8 __attribute__((ext_vector_type(8)));
typedef float f4 __attribute__((ext_vector_type(4)));
typedef uint32_t u4v __attribute__((ext_vector_type(4)));

constexpr int TOK = 32;        // tokens per KV block this kernel is built for
constexpr float TWO24 = 16777216.0f;
constexpr float LOG2E = 1.4426950408889634f;

__device__ inline uint32_t perm(uint32_t hi, uint32_t lo, uint32_t sel) { return __builtin_amdgcn_perm(hi, lo, sel); }

// bytes (e0 e1 e2 e3) of `w` -> two dwords of fp16 pairs (e0,e1) and (e2,e3), each byte zero-extended
__device__ inline void bytes_to_half_pairs(uint32_t w, uint32_t& p01, uint32_t& p23) {
    p01 = perm(0u, w, 0x0c010c00u);
    p23 = perm(0u, w, 0x0c030c02u);
}

// Reductions over the four 16-lane groups with the gfx950 lane-swap instructions (no LDS round trip):
// v_permlane16_swap exchanges the odd 16-lane rows of its first operand with the even rows of the second,
// v_permlane32_swap the upper half of the first with the lower half of the second; with both operands holding the
// same value the pair afterwards holds, per lane, the two values to combine.
__device__ __forceinline__ void swap_rows16(float& a, float& b) {
    asm volatile("s_nop 1\n\tv_permlane16_swap_b32 %0, %1\n\ts_nop 1" : "+v"(a), "+v"(b));
}
__device__ __forceinline__ void swap_halves32(float& a, float& b) {
    asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1\n\ts_nop 1" : "+v"(a), "+v"(b));
}
__device__ inline float xor_reduce_max_g(float v) {
    float a = v, b = v;
    swap_rows16(a, b);
    a = b = fmaxf(a, b);
    swap_halves32(a, b);
    return fmaxf(a, b);
}
__device__ inline float xor_reduce_sum_g(float v) {
    float a = v, b = v;
    swap_rows16(a, b);
    a = b = a + b;
    swap_halves32(a, b);
    return a + b;
}

// Loads one 32-token tile of K and V: whole-wave 16-byte passes plus the 16-chunk tails (K on lanes 0-15, V on 16-31).
// With 32-token cache blocks the tile is the block `phys0`; with 16-token blocks its halves are the blocks `phys0` and
// `phys1`, and each 16-byte chunk comes from the block its row lies in (the LDS image is the same).
// `sub`: with cache blocks of 64 tokens or more, which 32-token part of the block `phys0` the tile is (0 otherwise).
template <int FULL, int BS>
__device__ __forceinline__ void issue_block(const DecodeArgs& a, int phys0, int phys1, int sub, int hkv, int tile_bytes, int lane,
                                            u4v (&kraw)[FULL], u4v (&vraw)[FULL], u4v& traw) {
    if (BS == TOK) {
        const long base = ((long)phys0 * a.sh.Hkv + hkv) * ((long)tile_bytes * (a.sh.bs >> 5)) + (long)sub * tile_bytes;
        const u4v* kp = reinterpret_cast<const u4v*>(a.key_cache + base);
        const u4v* vp = reinterpret_cast<const u4v*>(a.value_cache + base);
#pragma unroll
        // every cache byte is used once per launch: streaming (non-temporal) loads keep it from displacing L2 contents
        for (int c = 0; c < FULL; ++c) {
            kraw[c] = __builtin_nontemporal_load(kp + c * 64 + lane);
            vraw[c] = __builtin_nontemporal_load(vp + c * 64 + lane);
        }
        traw = __builtin_nontemporal_load(((lane & 16) ? vp : kp) + FULL * 64 + (lane & 15));
    } else {
        const int half = tile_bytes / 2, half_chunks = half / 16;  // the tails lie in the second half
        const long base0 = ((long)phys0 * a.sh.Hkv + hkv) * half;
        const long base1 = ((long)phys1 * a.sh.Hkv + hkv) * half - half;
#pragma unroll
        for (int c = 0; c < FULL; ++c) {
            const int ci = c * 64 + lane;
            const long off = (ci < half_chunks ? base0 : base1) + (long)ci * 16;
            kraw[c] = __builtin_nontemporal_load(reinterpret_cast<const u4v*>(a.key_cache + off));
            vraw[c] = __builtin_nontemporal_load(reinterpret_cast<const u4v*>(a.value_cache + off));
        }
        const long toff = base1 + (long)(FULL * 64 + (lane & 15)) * 16;
        traw = __builtin_nontemporal_load(reinterpret_cast<const u4v*>(((lane & 16) ? a.value_cache : a.key_cache) + toff));
    }
}

template <int D, int QDT, int WAVES, int BS>
// (head size 256: one workgroup per CU, whose waves may then use the accumulation registers as well -- 16 KB blocks,
// two of them in flight, 64 accumulators and 32 query registers do not fit 256 registers)
__global__ __launch_bounds__(64 * WAVES, D > 128 ? 1 : 2) void pa_decode_u8_kernel(DecodeArgs a) {
    constexpr int BPT = TOK / BS;          // cache blocks per 32-token tile
    static_assert(BS == 32 || (BS == 16 && WAVES == 4), "the descriptor holds the ids of the first eight tiles");
    // BS = 32 stands for every block size from 32 tokens up (a power of two): a tile is then one 32-token part of a
    // block, the table slice in LDS holds the block id of every tile, and the part follows from the tile's number
    const int sub_mask = BS == 32 ? (a.sh.bs >> 5) - 1 : 0;
    const int sub_shift = BS == 32 ? 31 - __builtin_clz(a.sh.bs >> 5) : 0;
    const int bsz = BS == 32 ? a.sh.bs : BS;
    constexpr int NT = 64 * WAVES;
    constexpr int ROW = D + 8;
    constexpr int TILE = TOK * ROW;        // bytes of one (block, head) of K or V
    constexpr int FULL = TILE / 1024;      // whole-wave 16-byte passes; 16 chunks remain
    constexpr int KS = D / 32;             // k-steps of the QK contraction
    constexpr int RT = D / 16;             // 16-row output tiles of PV
    constexpr int VB = D / 16;             // V bytes per lane per token row
    constexpr int NW = (VB + 3) / 4;       // ... held in this many 32-bit words
    constexpr int SLOT = TILE;             // a wave's LDS staging slot: a K block, then a V block
    constexpr int EPL = (D + 63) / 64;     // elements per lane of a new K / V row
    constexpr int ROW_LANES = D / EPL;     // lanes a new row spreads over (D = 96: 48, the others repeat lanes 32 - 47)
    constexpr int DEPTH = 2;               // blocks a wave keeps in flight
    // Channel of row m of output tile r (the lane with n = m reads that channel's byte of each of its token rows): a
    // lane's VB consecutive channels, except that with 6 bytes per lane (D = 96) the lanes take four consecutive
    // channels of the first 64 and two of the last 32, so that their reads stay aligned.
    auto chan = [](const int m, const int r) __attribute__((always_inline)) {
        return D == 96 ? (r < 4 ? 4 * m + r : 64 + 2 * m + (r - 4)) : VB * m + r;
    };
    static_assert(TILE == FULL * 1024 + 256, "tile = whole passes + 16 chunks");
    extern __shared__ __align__(16) uint8_t smem[];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wv = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int n = lane & 15, g = lane >> 4;
    const StepDev& st = a.st;
    const int Hq = a.sh.Hq, Hkv = a.sh.Hkv, G = a.G, nsplit = a.nsplit;

    // grid = (split, kv head, listed sequence)
    const int split = blockIdx.x, hkv = blockIdx.y;
    // everything the first block fetches depend on sits in one descriptor (one scalar load)
    const DecodeDesc* __restrict__ dsc = a.descs + ((long)blockIdx.z * nsplit + split);
    const int b = dsc->b, t = dsc->t, kv_len = dsc->kv_len, first = dsc->first;
    const int tb = dsc->tb, te = dsc->te;
    const int tile_hi = (kv_len + TOK - 1) / TOK;
    const int32_t* table = a.block_indices + dsc->table_off;

    // LDS carve-up
    uint8_t* slot = smem + wv * SLOT;                                  // wave-private staging
    float* wave_mlz = reinterpret_cast<float*>(smem + WAVES * SLOT);   // [WAVES][16][4]
    float* msnap = wave_mlz + WAVES * 16 * 4;                          // [max_tiles][16]
    _Float16* ptile = reinterpret_cast<_Float16*>(msnap + (a.want_scores ? a.max_tiles * 16 : 0));  // [G][max_tiles*TOK]
    const int pstride = a.max_tiles * TOK;

    // The step's new K / V row of this (sequence, kv head) goes into the caches here when the step's append is fused
    // into this launch: by the wave that later reads the sequence's last block.  That wave's loads of the block must
    // see the row, and loads and stores of a wave may complete out of order with respect to each other, so the wave
    // waits for its stores explicitly (vmcnt(0)) before it issues the fetch of that block: at once when the block is
    // among its first ones, else (the stores then follow its first fetches) right in front of that fetch.
    const bool appends = a.fuse_append && te == tile_hi && te > tb && (tile_hi - 1 - tb) % WAVES == wv;
    const bool append_first = appends && tile_hi - 1 - tb < 4 * WAVES;
    auto append_rows = [&]() __attribute__((always_inline)) {
        const int rl = lane < ROW_LANES ? lane : lane - (64 - ROW_LANES);
        const long src = ((long)t * Hkv + hkv) * D + rl * EPL;
        const long dst = (((long)dsc->last_id * Hkv + hkv) * bsz + (kv_len - 1) % bsz) * ROW;
        uint16_t kr[EPL], vr[EPL];
        load_row16<EPL>(a.key + src, kr);
        load_row16<EPL>(a.value + src, vr);
        quantize_row_u8<QDT, EPL>(kr, const_cast<uint8_t*>(a.key_cache) + dst, rl, lane < ROW_LANES);
        quantize_row_u8<QDT, EPL>(vr, const_cast<uint8_t*>(a.value_cache) + dst, rl, lane < ROW_LANES);
    };
    if (append_first) {
        append_rows();
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    }

    // the first two blocks' loads go out before anything else is fetched
    u4v kraw[FULL], vraw[FULL], traw, kraw2[FULL], vraw2[FULL], traw2;
    int tile = tb + wv;
    if (tile < te)
        issue_block<FULL, BS>(a, dsc->ids[BPT * wv], dsc->ids[BPT * wv + BPT - 1], tile & sub_mask, hkv, TILE, lane, kraw, vraw, traw);
    if (DEPTH == 2 && tile + WAVES < te)
        issue_block<FULL, BS>(a, dsc->ids[BPT * (wv + WAVES)], dsc->ids[BPT * (wv + WAVES) + BPT - 1], (tile + WAVES) & sub_mask,
                              hkv, TILE, lane, kraw2, vraw2, traw2);
    const bool append_late = appends && !append_first;
    if (append_late) append_rows();
    // this workgroup's slice of the block table, so that no later block fetch waits on a table fetch
    int32_t* tab = reinterpret_cast<int32_t*>(smem + a.table_off);
    // (16-token blocks: two ids per tile; a last tile of one block repeats it, its second half lies beyond kv_len)
    {
        const int last_block = (kv_len + bsz - 1) / bsz - 1;
        for (int i = tid; i < BPT * (te - tb); i += NT) tab[i] = table[min((BPT * tb + i) >> sub_shift, last_block)];
    }

    // query operand (B of QK): lane (n, g) holds q[head n][32 s + 8 g + e]
    h8 qreg[KS];
    float qsum = 0.0f;
    {
        const uint16_t* qp = a.query + ((long)t * Hq + hkv * G + n) * D + 8 * g;
#pragma unroll
        for (int s = 0; s < KS; ++s) {
            if (n < G) {
                const uint4 v = *reinterpret_cast<const uint4*>(qp + 32 * s);
                if (QDT == DT_F16) {
                    qreg[s] = __builtin_bit_cast(h8, v);
                } else {
                    const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        qreg[s][2 * e] = (_Float16)bf16_bits_to_float((uint16_t)(w[e] & 0xffff));
                        qreg[s][2 * e + 1] = (_Float16)bf16_bits_to_float((uint16_t)(w[e] >> 16));
                    }
                }
            } else {
#pragma unroll
                for (int e = 0; e < 8; ++e) qreg[s][e] = (_Float16)0.0f;
            }
#pragma unroll
            for (int e = 0; e < 8; ++e) qsum += (float)qreg[s][e];
        }
        qsum = xor_reduce_sum_g(qsum);
    }
    const float scl24 = st.scale * LOG2E * TWO24;  // logits are kept in the log2 domain
    const float qsum24 = qsum * (1.0f / TWO24);

    float m_run = -INFINITY, l_part = 0.0f, z_part = 0.0f;
    f4 acc[RT];
#pragma unroll
    for (int r = 0; r < RT; ++r) acc[r] = f4{0.0f, 0.0f, 0.0f, 0.0f};

    __syncthreads();  // block-table slice is in LDS
    // one block of this wave's share: the block sits in (kr, vr, tr); once both halves are staged in LDS the same
    // registers take the loads of the block two turns ahead, so two blocks per wave are always in flight
    auto process = [&](u4v (&kr)[FULL], u4v (&vr)[FULL], u4v& tr, const int tile) __attribute__((always_inline)) {
        // ---- K block into the slot ------------------------------------------------------------
#pragma unroll
        for (int c = 0; c < FULL; ++c) reinterpret_cast<u4v*>(slot)[c * 64 + lane] = kr[c];
        if (lane < 16) reinterpret_cast<u4v*>(slot)[FULL * 64 + lane] = tr;
        __builtin_amdgcn_wave_barrier();

        // ---- S^T[token][head] = K . Q^T ---------------------------------------------------------
        f4 sc0 = f4{0.0f, 0.0f, 0.0f, 0.0f}, sc1 = f4{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int s = 0; s < KS; ++s) {
            const uint2 w0 = *reinterpret_cast<const uint2*>(slot + ROW * n + 8 + 32 * s + 8 * g);
            const uint2 w1 = *reinterpret_cast<const uint2*>(slot + ROW * (16 + n) + 8 + 32 * s + 8 * g);
            u4v a0, a1;
            uint32_t x0, x1;
            bytes_to_half_pairs(w0.x, x0, x1); a0[0] = x0; a0[1] = x1;
            bytes_to_half_pairs(w0.y, x0, x1); a0[2] = x0; a0[3] = x1;
            bytes_to_half_pairs(w1.x, x0, x1); a1[0] = x0; a1[1] = x1;
            bytes_to_half_pairs(w1.y, x0, x1); a1[2] = x0; a1[3] = x1;
            sc0 = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(h8, a0), qreg[s], sc0, 0, 0, 0);
            sc1 = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(h8, a1), qreg[s], sc1, 0, 0, 0);
        }
        // headers of this lane's eight tokens: token(u, i) = 16 u + 4 g + i
        float2 hk[8];
#pragma unroll
        for (int j = 0; j < 8; ++j)
            hk[j] = *reinterpret_cast<const float2*>(slot + ROW * (16 * (j >> 2) + 4 * g + (j & 3)));
        __builtin_amdgcn_wave_barrier();

        // ---- V block into the slot, next block's loads into flight -----------------------------
#pragma unroll
        for (int c = 0; c < FULL; ++c) reinterpret_cast<u4v*>(slot)[c * 64 + lane] = vr[c];
        if (lane >= 16 && lane < 32) reinterpret_cast<u4v*>(slot)[FULL * 64 + lane - 16] = tr;
        if (append_late && tile + DEPTH * WAVES == tile_hi - 1) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // the appended row is in place
        if (tile + DEPTH * WAVES < te) {
            const int ti = BPT * (tile + DEPTH * WAVES - tb);
            issue_block<FULL, BS>(a, tab[ti], tab[ti + BPT - 1], (tile + DEPTH * WAVES) & sub_mask, hkv, TILE, lane, kr, vr, tr);
        }
        __builtin_amdgcn_wave_barrier();

        // ---- online softmax (log2 domain) -------------------------------------------------------
        // Rows outside [first, kv_len) may hold anything, headers included: blocks that reach beyond either end
        // mask them (EDGE); the blocks in between, nearly all of a long context, skip the tests and selects.
        h8 pb, pl;
        auto softmax = [&](auto edge_tag) __attribute__((always_inline)) {
            constexpr bool EDGE = decltype(edge_tag)::value;
            float x[8];
            bool seen[8];
            float mx = -INFINITY;
            const int pos0 = tile * TOK;
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const float raw = (j < 4) ? sc0[j & 3] : sc1[j & 3];
                const int pos = pos0 + 16 * (j >> 2) + 4 * g + (j & 3);
                // scale * sc_k * (q . codes - zp_k * sum(q)), the code products still carrying their 2^-24
                float v = (hk[j].x * scl24) * __builtin_fmaf(-hk[j].y, qsum24, raw);
                seen[j] = !EDGE || (pos < kv_len && pos >= first);
                v = seen[j] ? v : -INFINITY;
                x[j] = v;
                mx = fmaxf(mx, v);
            }
            mx = xor_reduce_max_g(mx);
            const float m_new = fmaxf(m_run, mx);
            const float corr = __builtin_amdgcn_exp2f(m_run - m_new);
            float2 hv[8];
#pragma unroll
            for (int j = 0; j < 8; ++j)
                hv[j] = *reinterpret_cast<const float2*>(slot + ROW * (16 * (j >> 2) + 4 * g + (j & 3)));
            float psum = 0.0f, zsum = 0.0f;
            _Float16 ph[8];
            float wf[8];
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const float p = __builtin_amdgcn_exp2f(x[j] - m_new);
                wf[j] = seen[j] ? p * hv[j].x : 0.0f;
                psum += p;
                pb[j] = (_Float16)wf[j];
                ph[j] = (_Float16)p;
            }
            // The weights are pinned in their registers: the compiler may otherwise form the f16 value twice (from the
            // f32 product, and with a mixed-precision multiply), and the two differ by one f16 step at a tie
            asm volatile("" : "+v"(pb));
            // what the rounding to f16 dropped goes through the matrix pipe as a second operand: with 11 bits alone a
            // row that leans on a few tokens with large V values of opposite sign can miss the tolerance
#pragma unroll
            for (int j = 0; j < 8; ++j) pl[j] = (_Float16)(wf[j] - (float)pb[j]);
            asm volatile("" : "+v"(pl));
            // the zero-point term must see the weight the matrix product sees, or the rounding error is scaled by the
            // code instead of by (code - zp); the two halves together carry it to 2^-22, so the f32 weight serves
#pragma unroll
            for (int j = 0; j < 8; ++j) zsum += seen[j] ? wf[j] * hv[j].y : 0.0f;
            l_part = l_part * corr + psum;
            z_part = z_part * corr + zsum;
            m_run = m_new;
            if (__any(corr != 1.0f)) {
#pragma unroll
                for (int r = 0; r < RT; ++r) acc[r] *= corr;
            }
            if (a.want_scores) {
                const int lt = tile - tb;
                if (n < G) {
                    _Float16* dst = ptile + n * pstride + lt * TOK + 4 * g;
                    typedef _Float16 h4 __attribute__((ext_vector_type(4)));
                    *reinterpret_cast<h4*>(dst) = h4{ph[0], ph[1], ph[2], ph[3]};
                    *reinterpret_cast<h4*>(dst + 16) = h4{ph[4], ph[5], ph[6], ph[7]};
                    if (g == 0) msnap[lt * 16 + n] = m_new;
                }
            }
        };
        if (tile * TOK < first || tile * TOK + TOK > kv_len) softmax(std::true_type{});
        else softmax(std::false_type{});

        // ---- O^T[d][head] += V^T . P^T ----------------------------------------------------------
        // lane (m = n, g) reads the bytes of its channels chan(m, 0 .. VB - 1) of each of its eight token rows
        uint32_t vw[NW][8];
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const uint8_t* p = slot + ROW * (16 * (j >> 2) + 4 * g + (j & 3)) + 8;
            if constexpr (VB == 16) {  // (rows start on 8-byte boundaries)
                const uint2 w0 = *reinterpret_cast<const uint2*>(p + 16 * n);
                const uint2 w1 = *reinterpret_cast<const uint2*>(p + 16 * n + 8);
                vw[0][j] = w0.x, vw[1][j] = w0.y, vw[2][j] = w1.x, vw[3][j] = w1.y;
            } else if constexpr (VB == 8) {
                const uint2 w = *reinterpret_cast<const uint2*>(p + 8 * n);
                vw[0][j] = w.x, vw[1][j] = w.y;
            } else if constexpr (VB == 6) {
                vw[0][j] = *reinterpret_cast<const uint32_t*>(p + 4 * n);
                vw[1][j] = *reinterpret_cast<const uint16_t*>(p + 64 + 2 * n);
            } else {
                vw[0][j] = *reinterpret_cast<const uint32_t*>(p + 4 * n);
            }
        }
#pragma unroll
        for (int r = 0; r < RT; ++r) {
            const uint32_t sel = 0x0c000c00u | (uint32_t)(r & 3) | ((uint32_t)(4 + (r & 3)) << 16);
            u4v av;
#pragma unroll
            for (int p = 0; p < 4; ++p) av[p] = perm(vw[r >> 2][2 * p + 1], vw[r >> 2][2 * p], sel);
            acc[r] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(h8, av), pb, acc[r], 0, 0, 0);
            acc[r] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(h8, av), pl, acc[r], 0, 0, 0);
        }
        __builtin_amdgcn_wave_barrier();
    };
    for (; tile < te; tile += DEPTH * WAVES) {
        process(kraw, vraw, traw, tile);
        if (DEPTH == 2 && tile + WAVES < te) process(kraw2, vraw2, traw2, tile + WAVES);
    }

    // ---- merge the waves ---------------------------------------------------------------------------
    // Every wave leaves (max, denominator, zero-point sum) per head and its raw accumulators of the group's heads
    // (lanes n < G) in LDS; after one barrier each thread folds the waves for two channels of one head.
    const float l_w = xor_reduce_sum_g(l_part);
    const float z_w = xor_reduce_sum_g(z_part);
    __syncthreads();  // staging slots are dead from here on
    if (g == 0) {
        wave_mlz[(wv * 16 + n) * 4 + 0] = m_run;
        wave_mlz[(wv * 16 + n) * 4 + 1] = l_w;
        wave_mlz[(wv * 16 + n) * 4 + 2] = z_w;
    }
    // folds the waves' (m, l, z) of one head: the maximum, each wave's factor, denominator and zero-point sum
    auto fold_head = [&](const int head, float (&f)[WAVES], float& M, float& L, float& Z) __attribute__((always_inline)) {
        M = -INFINITY;
#pragma unroll
        for (int w = 0; w < WAVES; ++w) M = fmaxf(M, wave_mlz[(w * 16 + head) * 4]);
        L = 0.0f;
        Z = 0.0f;
#pragma unroll
        for (int w = 0; w < WAVES; ++w) {
            const float mw = wave_mlz[(w * 16 + head) * 4];
            f[w] = (mw == -INFINITY) ? 0.0f : __builtin_amdgcn_exp2f(mw - M);
            L += wave_mlz[(w * 16 + head) * 4 + 1] * f[w];
            Z += wave_mlz[(w * 16 + head) * 4 + 2] * f[w];
        }
    };
    // accumulators: [WAVES][HC][D] floats in the dead staging area, HC heads at a time
    constexpr int HC = 8;
    static_assert((size_t)WAVES * HC * D * sizeof(float) <= (size_t)WAVES * SLOT, "accumulators of a pass fit the staging area");
    float* red = reinterpret_cast<float*>(smem);
    const bool final_out = nsplit == 1;
    for (int n0 = 0; n0 < G; n0 += HC) {
        if (n0) __syncthreads();
        if (n >= n0 && n < min(G, n0 + HC)) {
            float* dst = red + ((wv * HC + n - n0) * D);
#pragma unroll
            for (int r = 0; r < RT; ++r)
#pragma unroll
                for (int i = 0; i < 4; ++i) dst[chan(4 * g + i, r)] = acc[r][i];  // lane (n, g), register i of tile r: row 4 g + i
        }
        __syncthreads();
        if (n0 == 0 && a.want_scores) {
            // one factor per (block, head): exp2(snapshot - M) (/ L when this workgroup saw the whole context), written
            // over the snapshot.  Entry e belongs to head e % 16 = this thread's n; the barrier before the score
            // phase publishes the factors
            float f[WAVES], M, L, Z;
            fold_head(n, f, M, L, Z);
            const float fl = final_out ? (L > 0.0f ? 1.0f / L : 0.0f) : 1.0f;
            for (int e = tid; e < max(te - tb, 0) * 16; e += NT)
                msnap[e] = n < G ? __builtin_amdgcn_exp2f(msnap[e] - M) * fl : 0.0f;
        }
        const int heads = min(G, n0 + HC) - n0;
        for (int idx = tid; idx < heads * (D / 2); idx += NT) {
            const int hl = idx / (D / 2), d = 2 * (idx % (D / 2));
            const int head = n0 + hl, hq = hkv * G + head;
            float f[WAVES], M, L, Z;
            fold_head(head, f, M, L, Z);
            float v0 = 0.0f, v1 = 0.0f;
#pragma unroll
            for (int w = 0; w < WAVES; ++w) {
                const float2 v = *reinterpret_cast<const float2*>(red + (w * HC + hl) * D + d);
                v0 += v.x * f[w];
                v1 += v.y * f[w];
            }
            const float o0 = v0 * TWO24 - Z, o1 = v1 * TWO24 - Z;
            const long prow = ((long)t * Hq + hq) * nsplit + split;
            if (final_out) {
                const float inv_l = L > 0.0f ? 1.0f / L : 0.0f;
                *reinterpret_cast<uint32_t*>(a.out + ((long)t * Hq + hq) * D + d) =
                    (uint32_t)store16<QDT>(o0 * inv_l) | ((uint32_t)store16<QDT>(o1 * inv_l) << 16);
            } else {
                *reinterpret_cast<float2*>(a.part_acc + prow * D + d) = make_float2(o0, o1);
            }
            if (d == 0) {  // maxima stay in the log2 domain within this kernel family
                float* ml = final_out ? a.final_ml + 2 * ((long)t * Hq + hq) : a.part_ml + 2 * prow;
                ml[0] = M;
                ml[1] = L;
            }
        }
    }

    // ---- scores: the factors were formed in place of the block maxima during the merge ---------------
    if (!a.want_scores) return;
    __syncthreads();
    const float* fac = msnap;
    typedef _Float16 h4 __attribute__((ext_vector_type(4)));
    typedef _Float16 h4u __attribute__((ext_vector_type(4), aligned(2)));
    const long soff = dsc->score_off;
    if (final_out) {
        // sum over the group's heads -> group_scores[hkv][position], four positions per thread, handed on as fp16
        // like the per-head probabilities of a launch with several splits (sums of at most 16 probabilities: the
        // rounding is 2^-12 of the value, and half the bytes go to HBM and come back);
        // positions before the first block of the window get 0
        _Float16* dst = a.group_scores + (long)hkv * a.total_scores + soff;
        const int p0 = tb * TOK;
        for (int pos = tid; pos < p0; pos += NT) dst[pos] = (_Float16)0.0f;
        const int cnt = kv_len - p0;
        for (int lp = 4 * tid; lp < cnt; lp += 4 * NT) {
            const float* f = fac + (lp / TOK) * 16;
            f4 sum = f4{0.0f, 0.0f, 0.0f, 0.0f};
            for (int h = 0; h < G; ++h) {
                const h4 p4 = *reinterpret_cast<const h4*>(ptile + h * pstride + lp);
                const float fh = f[h];
                sum[0] += (float)p4[0] * fh;
                sum[1] += (float)p4[1] * fh;
                sum[2] += (float)p4[2] * fh;
                sum[3] += (float)p4[3] * fh;
            }
            if (lp + 4 <= cnt) {
                *reinterpret_cast<h4u*>(dst + p0 + lp) = h4{(_Float16)sum[0], (_Float16)sum[1], (_Float16)sum[2], (_Float16)sum[3]};
            } else {
                for (int i = 0; lp + i < cnt; ++i) dst[p0 + lp + i] = (_Float16)sum[i];
            }
        }
    } else {
        // per-head probabilities relative to this split's maximum, fp16: p_split[hq][position], four positions per
        // thread (whole groups of four: the few values beyond kv_len land in the run's padding and are never used)
        const int p_lo = tb * TOK, p_hi = min(te * TOK, kv_len);
        const long stride = p_split_stride(a.total_scores, st.B), aoff = p_split_offset(soff, b);
        for (int h = 0; h < G; ++h) {
            _Float16* dst = a.p_split + (long)(hkv * G + h) * stride + aoff;
            for (int pos = p_lo + 4 * tid; pos < p_hi; pos += 4 * NT) {
                const int lp = pos - p_lo;
                const float fh = fac[(lp / TOK) * 16 + h];
                const h4 p4 = *reinterpret_cast<const h4*>(ptile + h * pstride + lp);
                *reinterpret_cast<h4*>(dst + pos) = h4{(_Float16)((float)p4[0] * fh), (_Float16)((float)p4[1] * fh),
                                                       (_Float16)((float)p4[2] * fh), (_Float16)((float)p4[3] * fh)};
            }
        }
    }
}

// Rows a launch's merge has to fold: every (token, head) of a step of single-token sequences, or those of the listed
// sequences of a mixed step.
__host__ __device__ inline long decode_merge_rows(const DecodeArgs& a) {
    return (long)(a.seq_list ? a.n_seqs : a.st.T) * a.sh.Hq;
}

// Folds split partials (log2 domain) into the output row and the final (max, denominator); `r` counts the launch's rows.
// WRITE_FAC: leave exp2(m_split - M) / L in place of the split denominators (for a score kernel that runs afterwards).
template <int D, int QDT, bool WRITE_FAC>
__device__ __forceinline__ void merge_row(const DecodeArgs& a, const long r, const int lane) {
    constexpr int EPL = (D + 63) / 64;  // (D = 96: two channels on each of the first 48 lanes)
    const bool act = lane * EPL < D;
    const int ch = act ? lane * EPL : 0;
    if (r >= decode_merge_rows(a)) return;
    long row = r;
    if (a.seq_list) {  // mixed step: the rows of the listed single-token sequences (the others are another kernel's)
        const int i = (int)(r / a.sh.Hq);
        row = (long)a.st.subsequence_begins[a.seq_list[i]] * a.sh.Hq + (r - (long)i * a.sh.Hq);
    }
    float M, inv, L;
    float acc[EPL];
#pragma unroll
    for (int e = 0; e < EPL; ++e) acc[e] = 0.0f;
    if (a.nsplit <= WAVE) {
        // lane s holds split s: one round of loads instead of a dependent chain
        const bool has = lane < a.nsplit;
        const float2 ml = has ? *reinterpret_cast<const float2*>(a.part_ml + 2 * (row * a.nsplit + lane))
                              : make_float2(-INFINITY, 0.0f);
        M = wave_max(ml.x);
        const float f_mine = ml.x == -INFINITY ? 0.0f : __builtin_amdgcn_exp2f(ml.x - M);
        L = wave_sum(ml.y * f_mine);
        inv = L > 0.0f ? 1.0f / L : 0.0f;
        // eight splits per round, loaded unconditionally (indices clamped, surplus ones weighted zero) so that
        // a round's loads are in flight together
        for (int s0 = 0; s0 < a.nsplit; s0 += 8) {
            float ms[8], v[8][EPL];
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const long slot = row * a.nsplit + min(s0 + j, a.nsplit - 1);
                ms[j] = a.part_ml[2 * slot];  // same address in every lane: one broadcast load
                const float* pa = a.part_acc + slot * D + ch;
#pragma unroll
                for (int e = 0; e < EPL; ++e) v[j][e] = pa[e];
            }
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const float f = (s0 + j >= a.nsplit || ms[j] == -INFINITY) ? 0.0f : __builtin_amdgcn_exp2f(ms[j] - M);
#pragma unroll
                for (int e = 0; e < EPL; ++e) acc[e] = fmaf(f == 0.0f ? 0.0f : v[j][e], f, acc[e]);  // empty splits hold nothing
            }
        }
        // the split denominators are spent: their places take the factor that turns a split's probabilities into
        // final ones, exp2(m_split - M) / L, for the score kernel
        if (WRITE_FAC && has) a.part_ml[2 * (row * a.nsplit + lane) + 1] = f_mine * inv;
    } else {
        M = -INFINITY;
        for (int s = 0; s < a.nsplit; ++s) M = fmaxf(M, a.part_ml[2 * (row * a.nsplit + s)]);
        L = 0.0f;
        for (int s = 0; s < a.nsplit; ++s) {
            const long slot = row * a.nsplit + s;
            const float ms = a.part_ml[2 * slot];
            if (ms == -INFINITY) continue;
            const float f = __builtin_amdgcn_exp2f(ms - M);
            L += a.part_ml[2 * slot + 1] * f;
#pragma unroll
            for (int e = 0; e < EPL; ++e) acc[e] += a.part_acc[slot * D + ch + e] * f;
        }
        inv = L > 0.0f ? 1.0f / L : 0.0f;
        for (int s = lane; WRITE_FAC && s < a.nsplit; s += WAVE) {
            const long slot = row * a.nsplit + s;
            const float ms = a.part_ml[2 * slot];
            a.part_ml[2 * slot + 1] = ms == -INFINITY ? 0.0f : __builtin_amdgcn_exp2f(ms - M) * inv;
        }
    }
#pragma unroll
    for (int e = 0; e < EPL; ++e)
        if (act) a.out[row * D + ch + e] = store16<QDT>(acc[e] * inv);
    if (lane == 0) {
        a.final_ml[2 * row] = M;
        a.final_ml[2 * row + 1] = L;
    }
}

template <int D, int QDT>
__global__ __launch_bounds__(256) void pa_decode_merge_kernel(DecodeArgs a) {
    merge_row<D, QDT, true>(a, (long)blockIdx.x * 4 + (threadIdx.x >> 6), threadIdx.x & 63);
}

// scores[position] = sum over kv heads of the group sums, kv heads in ascending order (single split), or
// sum over query heads of p_split * exp2(m_split - M) / L (several splits; the factor comes from the merge kernel).
// W = 0 gives zeros.
// LDS_FAC: the split-to-final factors come from `s_fac` ([Hq][nsplit]) instead of the places the merge kernel wrote.
template <bool LDS_FAC>
__device__ __forceinline__ void score_positions(const DecodeArgs& a, float* __restrict__ scores, const int bx, const int gx,
                                                const int by, const float* s_fac) {
    const StepDev& st = a.st;
    const int b = a.seq_list ? a.seq_list[by] : by;
    const int kv_len = st.past_lens[b] + 1;
    const long soff = st.score_offsets[b];
    const int t = st.subsequence_begins[b];
    const bool live = st.score_window[b] > 0;
    const int first = st.sliding_window > 0 ? max(0, kv_len - st.sliding_window) : 0;
    if (a.nsplit == 1) {
        for (int pos = bx * 256 + threadIdx.x; pos < kv_len; pos += gx * 256) {
            float s = 0.0f;
            if (live && pos >= first) {
#pragma unroll 8
                for (int h = 0; h < a.sh.Hkv; ++h) s += (float)a.group_scores[(long)h * a.total_scores + soff + pos];
            }
            scores[soff + pos] = s;
        }
        return;
    }
    // several splits: eight positions per thread (one 16-byte load per head); a group of eight lies inside one KV
    // block, hence inside one split
    typedef _Float16 h8v __attribute__((ext_vector_type(8)));
    const int tile_lo = first / TOK, tile_hi = (kv_len + TOK - 1) / TOK;
    const int per = ceil_div(tile_hi - tile_lo, a.nsplit);
    const long stride = p_split_stride(a.total_scores, st.B), aoff = p_split_offset(soff, b);
    for (int p8 = (bx * 256 + threadIdx.x) * 8; p8 < kv_len; p8 += gx * 256 * 8) {
        float s[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) s[i] = 0.0f;
        if (live && p8 + 7 >= first) {
            const int split = (p8 / TOK - tile_lo) / per;
            const float* fac = a.part_ml + 2 * ((long)t * a.sh.Hq * a.nsplit + split) + 1;  // + 2 * nsplit per head
            const _Float16* p = a.p_split + aoff + p8;
#pragma unroll 8
            for (int h = 0; h < a.sh.Hq; ++h) {  // unrolled: several heads' loads in flight together
                const float f = LDS_FAC ? s_fac[h * a.nsplit + split] : fac[2L * h * a.nsplit];
                const h8v v = *reinterpret_cast<const h8v*>(p + h * stride);
#pragma unroll
                for (int i = 0; i < 8; ++i) s[i] = fmaf((float)v[i], f, s[i]);
            }
        }
#pragma unroll
        for (int i = 0; i < 8; ++i)
            if (p8 + i < kv_len) scores[soff + p8 + i] = (live && p8 + i >= first) ? s[i] : 0.0f;
    }
}

__global__ __launch_bounds__(256) void pa_decode_scores_kernel(DecodeArgs a, float* __restrict__ scores) {
    score_positions<false>(a, scores, blockIdx.x, gridDim.x, blockIdx.y, nullptr);
}

// Merge and scores of a launch with several splits in one launch: the first `merge_blocks` workgroups fold the split
// partials into output rows (four rows each); the others take (sequence, range of positions) and form the
// split-to-final factors of their sequence's heads themselves, in LDS, so neither role waits for the other.
template <int D, int QDT>
__global__ __launch_bounds__(256) void pa_decode_post_kernel(DecodeArgs a, float* __restrict__ scores, int merge_blocks,
                                                             int gx) {
    extern __shared__ float s_fac[];  // [Hq][nsplit] factors, then [Hq][nsplit] (maximum, denominator) pairs
    const int id = blockIdx.x;
    if (id < merge_blocks) {
        merge_row<D, QDT, false>(a, (long)id * 4 + (threadIdx.x >> 6), threadIdx.x & 63);
        return;
    }
    const int sid = id - merge_blocks, bx = sid % gx, by = sid / gx;
    const int b = a.seq_list ? a.seq_list[by] : by;
    const int t = a.st.subsequence_begins[b];
    // the sequence's (maximum, denominator) pairs, one per (head, split): every thread fetches its share with all
    // loads in flight, then one thread per head folds its row out of LDS (a thread per head reading its row from
    // global memory walked a chain of dependent loads: 3.5 us more on a step of one sequence)
    const int n_pairs = a.sh.Hq * a.nsplit;
    float2* s_ml = reinterpret_cast<float2*>(s_fac + n_pairs);  // [Hq][nsplit]
    const float2* ml_g = reinterpret_cast<const float2*>(a.part_ml) + (long)t * n_pairs;
    for (int i0 = threadIdx.x; i0 < n_pairs; i0 += 4 * 256) {
        float2 v[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) v[j] = ml_g[min(i0 + 256 * j, n_pairs - 1)];
#pragma unroll
        for (int j = 0; j < 4; ++j)
            if (i0 + 256 * j < n_pairs) s_ml[i0 + 256 * j] = v[j];
    }
    __syncthreads();
    for (int h = threadIdx.x; h < a.sh.Hq; h += 256) {
        const float2* ml = s_ml + h * a.nsplit;
        float M = -INFINITY, L = 0.0f;
        for (int s = 0; s < a.nsplit; ++s) M = fmaxf(M, ml[s].x);
        for (int s = 0; s < a.nsplit; ++s)
            if (ml[s].x != -INFINITY) L += ml[s].y * __builtin_amdgcn_exp2f(ml[s].x - M);
        const float inv = L > 0.0f ? 1.0f / L : 0.0f;
        for (int s = 0; s < a.nsplit; ++s)
            s_fac[h * a.nsplit + s] = ml[s].x == -INFINITY ? 0.0f : __builtin_amdgcn_exp2f(ml[s].x - M) * inv;
    }
    __syncthreads();
    score_positions<true>(a, scores, bx, gx, by, s_fac);
}

}  // namespace

// LDS layout: staging | per-wave (m, l, z) | [scores: block maxima | probabilities] | block-table slice
size_t decode_u8_lds_bytes(int D, int G, int max_tiles, bool want_scores, int waves, int32_t* table_off, int block_size) {
    size_t bytes = (size_t)waves * TOK * (D + 8) + waves * 16 * 4 * sizeof(float);
    if (want_scores) bytes += (size_t)max_tiles * 16 * sizeof(float) + (size_t)G * max_tiles * TOK * sizeof(uint16_t);
    bytes = (bytes + 15) & ~(size_t)15;
    *table_off = (int32_t)bytes;
    bytes += (size_t)max_tiles * (block_size == 16 ? 2 : 1) * sizeof(int32_t);
    return (bytes + 15) & ~(size_t)15;
}

template <int D, int QDT, int WAVES, int BS>
static hipError_t launch_decode_typed(hipStream_t s, const DecodeArgs& a_in, float* scores, int max_kv_len,
                                      hipEvent_t ev0, hipEvent_t ev1) {
    DecodeArgs a = a_in;
    const size_t lds = decode_u8_lds_bytes(D, a.G, a.max_tiles, a.want_scores != 0, WAVES, &a.table_off, BS);
    auto kern = pa_decode_u8_kernel<D, QDT, WAVES, BS>;
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) return e;
    if (a.n_seqs > 65535) return hipErrorInvalidValue;  // grid z
    if (ev0) (void)hipEventRecord(ev0, s);
    hipLaunchKernelGGL(kern, dim3((unsigned)a.nsplit, (unsigned)a.sh.Hkv, (unsigned)a.n_seqs), dim3(64 * WAVES), lds, s, a);
    if (ev1) (void)hipEventRecord(ev1, s);
    return launch_decode_post(s, a, QDT, scores, max_kv_len);
}

template <int D, int QDT>
static hipError_t launch_decode_waves(hipStream_t s, const DecodeArgs& a, float* scores, int max_kv_len,
                                      hipEvent_t ev0, hipEvent_t ev1) {
    if (a.sh.bs == 16) {
        if (a.waves != 4) return hipErrorInvalidValue;
        return launch_decode_typed<D, QDT, 4, 16>(s, a, scores, max_kv_len, ev0, ev1);
    }
    if (a.sh.bs < 32 || a.sh.bs > 256 || (a.sh.bs & (a.sh.bs - 1))) return hipErrorInvalidValue;
    if (a.waves == 8) {
        // (eight-wave workgroups leave a wave 128 registers: head sizes 64 and 128)
        if constexpr (D == 64 || D == 128) return launch_decode_typed<D, QDT, 8, 32>(s, a, scores, max_kv_len, ev0, ev1);
        else return hipErrorInvalidValue;
    }
    return launch_decode_typed<D, QDT, 4, 32>(s, a, scores, max_kv_len, ev0, ev1);
}

hipError_t launch_decode_scores(hipStream_t s, const DecodeArgs& a, float* scores, int max_kv_len) {
    const int per_wg = a.nsplit == 1 ? 256 : 2048;  // positions a workgroup covers per pass
    dim3 grid((unsigned)min(ceil_div(max_kv_len, per_wg), 64), (unsigned)a.n_seqs);
    hipLaunchKernelGGL(pa_decode_scores_kernel, grid, dim3(256), 0, s, a, scores);
    return hipGetLastError();
}

hipError_t launch_decode_merge(hipStream_t s, const DecodeArgs& a, int q_dtype) {
    const dim3 grid((unsigned)((decode_merge_rows(a) + 3) / 4));
#define PA_MERGE(D_)                                                                                              \
    if (a.sh.D == D_) {                                                                                           \
        if (q_dtype == DT_F16) hipLaunchKernelGGL((pa_decode_merge_kernel<D_, DT_F16>), grid, dim3(256), 0, s, a); \
        else hipLaunchKernelGGL((pa_decode_merge_kernel<D_, DT_BF16>), grid, dim3(256), 0, s, a);                  \
        return hipGetLastError();                                                                                 \
    }
    PA_MERGE(128)
    PA_MERGE(64)
    PA_MERGE(96)
    PA_MERGE(256)
#undef PA_MERGE
    return hipErrorInvalidValue;
}

template <int D, int QDT>
static hipError_t launch_post_typed(hipStream_t s, const DecodeArgs& a, float* scores, int max_kv_len) {
    const int gx = min(ceil_div(max_kv_len, 2048), 64);
    const int merge_blocks = (int)((decode_merge_rows(a) + 3) / 4);
    const size_t lds = (size_t)a.sh.Hq * a.nsplit * 3 * sizeof(float);
    hipLaunchKernelGGL((pa_decode_post_kernel<D, QDT>), dim3((unsigned)(merge_blocks + gx * a.n_seqs)), dim3(256), lds, s, a,
                       scores, merge_blocks, gx);
    return hipGetLastError();
}

// What follows a decode launch: with several splits the merge, with scores the score kernel, both in one launch when
// the factors of a sequence's heads fit a small LDS table.
hipError_t launch_decode_post(hipStream_t s, const DecodeArgs& a, int q_dtype, float* scores, int max_kv_len) {
    if (a.nsplit > 1 && scores && a.sh.Hq * a.nsplit <= 4096) {
#define PA_POST(D_)                                                                               \
    if (a.sh.D == D_)                                                                             \
        return q_dtype == DT_F16 ? launch_post_typed<D_, DT_F16>(s, a, scores, max_kv_len)       \
                                 : launch_post_typed<D_, DT_BF16>(s, a, scores, max_kv_len);
        PA_POST(128)
        PA_POST(64)
        PA_POST(96)
        PA_POST(256)
#undef PA_POST
    }
    hipError_t e;
    if (a.nsplit > 1 && (e = launch_decode_merge(s, a, q_dtype)) != hipSuccess) return e;
    return scores ? launch_decode_scores(s, a, scores, max_kv_len) : hipSuccess;
}

// The runtime uploads a translation unit's device code when one of its kernels is first asked for; asking here, when
// a context is created, keeps that allocation out of the first attention call.
hipError_t preload_decode_u8() {
    hipFuncAttributes at;
    return hipFuncGetAttributes(&at, reinterpret_cast<const void*>(pa_decode_u8_kernel<128, DT_F16, 4, 32>));
}

hipError_t launch_decode_u8(hipStream_t s, const DecodeArgs& a, int q_dtype, float* scores, int max_kv_len,
                            hipEvent_t ev0, hipEvent_t ev1) {
    if (a.sh.D == 128)
        return q_dtype == DT_F16 ? launch_decode_waves<128, DT_F16>(s, a, scores, max_kv_len, ev0, ev1)
                                 : launch_decode_waves<128, DT_BF16>(s, a, scores, max_kv_len, ev0, ev1);
    if (a.sh.D == 64)
        return q_dtype == DT_F16 ? launch_decode_waves<64, DT_F16>(s, a, scores, max_kv_len, ev0, ev1)
                                 : launch_decode_waves<64, DT_BF16>(s, a, scores, max_kv_len, ev0, ev1);
    if (a.sh.D == 96)
        return q_dtype == DT_F16 ? launch_decode_waves<96, DT_F16>(s, a, scores, max_kv_len, ev0, ev1)
                                 : launch_decode_waves<96, DT_BF16>(s, a, scores, max_kv_len, ev0, ev1);
    if (a.sh.D == 256)
        return q_dtype == DT_F16 ? launch_decode_waves<256, DT_F16>(s, a, scores, max_kv_len, ev0, ev1)
                                 : launch_decode_waves<256, DT_BF16>(s, a, scores, max_kv_len, ev0, ev1);
    return hipErrorInvalidValue;
}

}  // namespace pa
