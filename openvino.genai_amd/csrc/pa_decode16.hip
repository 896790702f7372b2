// Decode (q_len = 1) PagedAttention over a 16-bit KV cache (f16 or bf16, the query's type): the bandwidth-bound
// counterpart of the u8 decode kernel.
//
// Work item = (sequence, kv head, split): one 256-thread workgroup, four waves taking the split's 32-token KV blocks
// round-robin, each wave with its own running maximum / denominator / accumulators (merged at the end) -- through
// the matrix kernel a single-token sequence keeps one of eight waves busy with arithmetic while seven only move
// blocks.  Per block and wave:
//   * K rows go straight from global memory into MFMA A operands (lane (n, g): token 16 u + n, channels
//     32 s + 8 g .. + 7 -- 16 contiguous bytes), V rows with fully coalesced 16-byte loads into a wave-private LDS
//     slot and from there through the transposing LDS read into A operands; both one block ahead of the arithmetic;
//   * S^T[token][head] = K . Q^T and O^T[channel][head] += V^T . P^T on v_mfma_f32_16x16x32_{f16,bf16} with the GQA
//     group (<= 16 query heads sharing the kv head) as the N dimension: every cache byte is read once per group;
//   * P enters as hi + lo halves of the operand type (8 significant bits for bf16, 11 for f16, are not enough where
//     large V elements of opposite sign cancel);
//   * online softmax in the log2 domain per wave.
// Scores as in the u8 decode kernel: the un-normalised probabilities of a workgroup's positions stay in LDS (fp16,
// relative to the running maximum, which is snapshotted per block); once the final maximum and denominator are
// known they are normalised, summed over the group's heads and written out.
// Split partials, per-kv-head score sums and split probabilities have the layouts of the u8 decode kernel and are
// folded by its merge and score kernels.
//
// Roofline: HBM.  Algorithmic bytes per (sequence, kv head, position): 4 * D.
#include "pa_device.h"

namespace pa {
namespace {

typedef _Float16 h8 __attribute__((ext_vector_type(8)));
typedef __bf16 b8 __attribute__((ext_vector_type(8)));
typedef short s8v __attribute__((ext_vector_type(8)));
typedef short s4v __attribute__((ext_vector_type(4)));
typedef float f4 __attribute__((ext_vector_type(4)));
typedef uint32_t u4v __attribute__((ext_vector_type(4)));

constexpr int TOK = 32;
constexpr float LOG2E = 1.4426950408889634f;

template <int DT>
__device__ __forceinline__ f4 mma(const s8v& a, const s8v& b, const f4& c) {
    if (DT == DT_F16)
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(h8, a), __builtin_bit_cast(h8, b), c, 0, 0, 0);
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(b8, a), __builtin_bit_cast(b8, b), c, 0, 0, 0);
}

__device__ __forceinline__ s4v lds_read_tr16(const uint8_t* p) {
    typedef s4v __attribute__((address_space(3))) * lds_ptr;
    return __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)p);
}

template <int DT>
__device__ __forceinline__ uint32_t pack2(float a, float b) {
    if (DT == DT_F16) {
        typedef _Float16 h2 __attribute__((ext_vector_type(2)));
        return __builtin_bit_cast(uint32_t, h2{(_Float16)a, (_Float16)b});
    }
    typedef __bf16 b2 __attribute__((ext_vector_type(2)));
    return __builtin_bit_cast(uint32_t, b2{(__bf16)a, (__bf16)b});
}

__device__ __forceinline__ float group_max(float v) {  // over the four 16-lane groups
    v = fmaxf(v, __shfl_xor(v, 16, WAVE));
    return fmaxf(v, __shfl_xor(v, 32, WAVE));
}
__device__ __forceinline__ float group_sum(float v) {
    v += __shfl_xor(v, 16, WAVE);
    return v + __shfl_xor(v, 32, WAVE);
}

// (head size 256: one workgroup per CU, whose waves may then use the accumulation registers as well -- two 32 KB
// blocks in flight are 256 registers by themselves)
template <int D, int DT, int BS>
__global__ __launch_bounds__(256, D > 128 ? 1 : 2) void pa_decode16_kernel(DecodeArgs a) {
    constexpr int WAVES = 4;
    constexpr int BPT = TOK / BS;          // cache blocks per 32-token tile (with two, each holds one row group)
    // BS = 32 stands for every block size from 32 tokens up (a power of two): a tile is then one 32-token part of a block
    const int sub_mask = BS == 32 ? (a.sh.bs >> 5) - 1 : 0;
    const int sub_shift = BS == 32 ? 31 - __builtin_clz(a.sh.bs >> 5) : 0;
    const int bsz = BS == 32 ? a.sh.bs : BS;
    constexpr int ROWB = D * 2;            // bytes of a cache row
    constexpr int TILE = TOK * ROWB;       // bytes of one (block, head) of K or V
    constexpr int LROWV = ROWB + 32;       // LDS row stride of the V slot (the transposing reads are conflict free)
    constexpr int SLOT = TOK * LROWV;
    constexpr int KS = D / 32;             // k-steps of the QK contraction
    constexpr int RT = D / 16;             // 16-channel output tiles of PV
    constexpr int VCH = TILE / 1024;       // 16-byte pieces of the V block per lane
    constexpr int CPR = ROWB / 16;         // 16-byte pieces per row
    extern __shared__ __align__(16) uint8_t smem[];

    const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
    const int n = lane & 15, g = lane >> 4;
    const StepDev& st = a.st;
    const int Hq = a.sh.Hq, Hkv = a.sh.Hkv, G = a.G, nsplit = a.nsplit;
    const int split = blockIdx.x % nsplit;
    const int hkv = (blockIdx.x / nsplit) % Hkv;
    const int b = a.seq_list ? a.seq_list[blockIdx.x / (nsplit * Hkv)] : (int)(blockIdx.x / (nsplit * Hkv));
    const int t = st.subsequence_begins[b];
    const int kv_len = st.past_lens[b] + 1;
    const int first = st.sliding_window > 0 ? max(0, kv_len - st.sliding_window) : 0;
    const int tile_lo = first / TOK, tile_hi = (kv_len + TOK - 1) / TOK;
    const int per = ceil_div(tile_hi - tile_lo, nsplit);
    const int tb = tile_lo + split * per;
    const int te = min(tile_hi, tb + per);
    const int32_t* table = a.block_indices + st.block_indices_begins[b];

    uint8_t* slot = smem + wv * SLOT;                                  // this wave's V block
    float* wave_ml = reinterpret_cast<float*>(smem + WAVES * SLOT);    // [WAVES][16][2]
    float* msnap = wave_ml + WAVES * 16 * 2;                           // [max_tiles][G] running maximum at each block
    _Float16* ptile = reinterpret_cast<_Float16*>(msnap + (a.want_scores ? decode16_snap_floats(a.max_tiles, G) : 0));  // [G][max_tiles * TOK]
    const int pstride = a.max_tiles * TOK;
    int32_t* tab = reinterpret_cast<int32_t*>(smem + a.table_off);     // the workgroup's slice of the block table

    // one block's K operands and V pieces in registers
    struct Block {
        u4v k[2][KS];
        u4v v[VCH];
    };
    // the tile's two row groups: halves of the block `phys0`, or the 16-token blocks `phys0` and `phys1`
    auto issue = [&](Block& blk, int phys0, int phys1, int sub) __attribute__((always_inline)) {
        const long base0 = BS == TOK ? ((long)phys0 * Hkv + hkv) * ((long)TILE * (a.sh.bs >> 5)) + (long)sub * TILE
                                     : ((long)phys0 * Hkv + hkv) * (TILE / BPT);
        const long base1 = BS == TOK ? base0 + TILE / 2 : ((long)phys1 * Hkv + hkv) * (TILE / 2);
#pragma unroll
        for (int u = 0; u < 2; ++u)
#pragma unroll
            for (int s = 0; s < KS; ++s)
                blk.k[u][s] = __builtin_nontemporal_load(reinterpret_cast<const u4v*>(
                    a.key_cache + (u ? base1 : base0) + n * ROWB + (32 * s + 8 * g) * 2));
        static_assert(VCH % 2 == 0, "each half of the V tile is a whole number of wave passes");
#pragma unroll
        for (int c = 0; c < VCH; ++c)
            blk.v[c] = __builtin_nontemporal_load(reinterpret_cast<const u4v*>(
                           a.value_cache + (c < VCH / 2 ? base0 : base1 - TILE / 2)) + c * 64 + lane);
    };
    const int last_block = (kv_len + bsz - 1) / bsz - 1;  // a last tile of one 16-token block repeats it (rows masked)
    Block ba, bb;
    int tile = tb + wv;
    // The step's new K / V row of this (sequence, kv head) goes into the caches here when the step's append is fused
    // into this launch: by the wave that later reads the sequence's last tile, which waits for the two stores before
    // it fetches that tile (at once when it is the wave's first tile, else in front of the fetch, see `process`).
    const bool owner = a.fuse_append && te == tile_hi && te > tb && (tile_hi - 1 - tb) % WAVES == wv;
    auto append_row = [&]() __attribute__((always_inline)) {
        if (lane < 2 * CPR) {  // lanes 0 .. CPR-1: the K row's 16-byte pieces, the next CPR lanes: the V row's
            const bool isv = lane >= CPR;
            const int piece = isv ? lane - CPR : lane, pos = kv_len - 1;
            const u4v row = *reinterpret_cast<const u4v*>(reinterpret_cast<const uint8_t*>(isv ? a.value : a.key) +
                                                          ((long)t * Hkv + hkv) * ROWB + piece * 16);
            const long dst = (((long)table[pos / bsz] * Hkv + hkv) * bsz + pos % bsz) * ROWB + piece * 16;
            *reinterpret_cast<u4v*>(const_cast<uint8_t*>(isv ? a.value_cache : a.key_cache) + dst) = row;
        }
    };
    if (owner && tile == tile_hi - 1) {
        append_row();
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    }
    if (tile < te)
        issue(ba, table[min((BPT * tile) >> sub_shift, last_block)], table[min((BPT * tile + BPT - 1) >> sub_shift, last_block)],
              tile & sub_mask);
    if (owner && tile != tile_hi - 1) append_row();
    for (int i = tid; i < BPT * (te - tb); i += 64 * WAVES) tab[i] = table[min((BPT * tb + i) >> sub_shift, last_block)];

    // query operand (B of QK): lane (n, g) holds q[head n][32 s + 8 g + e]; heads beyond the group are zero
    s8v qreg[KS];
    {
        const uint16_t* qp = a.query + ((long)t * Hq + hkv * G + min(n, G - 1)) * D + 8 * g;
#pragma unroll
        for (int s = 0; s < KS; ++s) {
            const u4v v = *reinterpret_cast<const u4v*>(qp + 32 * s);
            qreg[s] = __builtin_bit_cast(s8v, n < G ? v : u4v{0u, 0u, 0u, 0u});
        }
    }
    const float scl = st.scale * LOG2E;
    float m_run = -INFINITY, l_part = 0.0f;
    f4 acc[RT];
#pragma unroll
    for (int r = 0; r < RT; ++r) acc[r] = f4{0.0f, 0.0f, 0.0f, 0.0f};
    __syncthreads();  // block-table slice is in LDS

    auto process = [&](Block& cur, Block& nxt, const int tl) __attribute__((always_inline)) {
        // next block's loads into flight, this block's V into the slot
        if (owner && tl + WAVES == tile_hi - 1) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // the appended row is in place
        if (tl + WAVES < te) issue(nxt, tab[BPT * (tl + WAVES - tb)], tab[BPT * (tl + WAVES - tb) + BPT - 1], (tl + WAVES) & sub_mask);
#pragma unroll
        for (int c = 0; c < VCH; ++c) {
            const int piece = c * 64 + lane;
            // rows beyond the sequence's last token may hold anything: zero them so that 0 * garbage cannot reach the
            // accumulators (their K columns are masked below)
            const bool live = tl * TOK + piece / CPR < kv_len;
            *reinterpret_cast<u4v*>(slot + (piece / CPR) * LROWV + (piece % CPR) * 16) = live ? cur.v[c] : u4v{0u, 0u, 0u, 0u};
        }
        // S^T[token][head] = K . Q^T
        f4 sc[2];
#pragma unroll
        for (int u = 0; u < 2; ++u) {
            sc[u] = f4{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
            for (int s = 0; s < KS; ++s) sc[u] = mma<DT>(__builtin_bit_cast(s8v, cur.k[u][s]), qreg[s], sc[u]);
        }
        // online softmax: lane (n, g) holds head n, tokens 16 u + 4 g + i
        float x[8];
        float mx = -INFINITY;
        const int pos0 = tl * TOK + 4 * g;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const int pos = pos0 + 16 * (j >> 2) + (j & 3);
            x[j] = (pos < kv_len && pos >= first) ? sc[j >> 2][j & 3] * scl : -INFINITY;
            mx = fmaxf(mx, x[j]);
        }
        mx = group_max(mx);
        const float m_new = fmaxf(m_run, mx);
        const float m_safe = m_new == -INFINITY ? 0.0f : m_new;
        const float corr = __builtin_amdgcn_exp2f(m_run - m_safe);
        float p[8], psum = 0.0f;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            p[j] = __builtin_amdgcn_exp2f(x[j] - m_safe);
            psum += p[j];
        }
        u4v pb, pl;
#pragma unroll
        for (int jj = 0; jj < 4; ++jj) {
            const uint32_t hi = pack2<DT>(p[2 * jj], p[2 * jj + 1]);
            pb[jj] = hi;
            if (DT == DT_BF16) {
                pl[jj] = pack2<DT>(p[2 * jj] - __builtin_bit_cast(float, hi << 16),
                                   p[2 * jj + 1] - __builtin_bit_cast(float, hi & 0xffff0000u));
            } else {
                typedef _Float16 h2 __attribute__((ext_vector_type(2)));
                const h2 h = __builtin_bit_cast(h2, hi);
                pl[jj] = pack2<DT>(p[2 * jj] - (float)h[0], p[2 * jj + 1] - (float)h[1]);
            }
        }
        l_part = l_part * corr + psum;
        m_run = m_new;
        if (__any(corr != 1.0f)) {
#pragma unroll
            for (int r = 0; r < RT; ++r) acc[r] *= corr;
        }
        if (a.want_scores) {
            const int lt = tl - tb;
            if (n < G) {
                typedef _Float16 h4 __attribute__((ext_vector_type(4)));
                _Float16* dst = ptile + n * pstride + lt * TOK + 4 * g;
                *reinterpret_cast<h4*>(dst) = h4{(_Float16)p[0], (_Float16)p[1], (_Float16)p[2], (_Float16)p[3]};
                *reinterpret_cast<h4*>(dst + 16) = h4{(_Float16)p[4], (_Float16)p[5], (_Float16)p[6], (_Float16)p[7]};
                if (g == 0) msnap[lt * G + n] = m_safe;
            }
        }
        __builtin_amdgcn_wave_barrier();  // the slot was written by this wave's own lanes
        // O^T[channel][head] += V^T . P^T: lane n of a group receives channel 16 r + n of tokens 16 h + 4 g + 0..3
#pragma unroll
        for (int r = 0; r < RT; ++r) {
            const uint8_t* p0 = slot + (4 * g + (n >> 2)) * LROWV + (16 * r + 4 * (n & 3)) * 2;
            const s4v v0 = lds_read_tr16(p0);
            const s4v v1 = lds_read_tr16(p0 + 16 * LROWV);
            const s8v vop = s8v{v0[0], v0[1], v0[2], v0[3], v1[0], v1[1], v1[2], v1[3]};
            acc[r] = mma<DT>(vop, __builtin_bit_cast(s8v, pb), acc[r]);
            acc[r] = mma<DT>(vop, __builtin_bit_cast(s8v, pl), acc[r]);
        }
        __builtin_amdgcn_wave_barrier();  // before the next block's V overwrites the slot
    };
    for (; tile < te; tile += 2 * WAVES) {
        process(ba, bb, tile);
        if (tile + WAVES < te) process(bb, ba, tile + WAVES);
    }

    // ---- merge the four waves ----------------------------------------------------------------------
    const float l_w = group_sum(l_part);
    __syncthreads();  // the V slots are dead from here on
    if (g == 0) {
        wave_ml[(wv * 16 + n) * 2] = m_run;
        wave_ml[(wv * 16 + n) * 2 + 1] = l_w;
    }
    __syncthreads();
    float M = -INFINITY;
#pragma unroll
    for (int w = 0; w < WAVES; ++w) M = fmaxf(M, wave_ml[(w * 16 + n) * 2]);
    float L = 0.0f;
#pragma unroll
    for (int w = 0; w < WAVES; ++w) {
        const float mw = wave_ml[(w * 16 + n) * 2];
        L += (mw == -INFINITY) ? 0.0f : wave_ml[(w * 16 + n) * 2 + 1] * __builtin_amdgcn_exp2f(mw - M);
    }
    const float f_own = (m_run == -INFINITY) ? 0.0f : __builtin_amdgcn_exp2f(m_run - M);
    // accumulators: [WAVES][RT / 2 tiles][4][64] floats in the dead V slots, half of the tiles at a time; wave w then
    // finishes the tiles r = w, w + WAVES, .. of the half
    float* red = reinterpret_cast<float*>(smem);
    constexpr int HALF = RT / 2;
    static_assert((size_t)WAVES * HALF * 4 * 64 * sizeof(float) <= (size_t)WAVES * SLOT, "the reduction fits the V slots");
    const bool final_out = nsplit == 1;
    const int hq = hkv * G + n;
    const long prow = ((long)t * Hq + hq) * nsplit + split;
    const float inv_l = L > 0.0f ? 1.0f / L : 0.0f;
    if (a.want_scores) {
        // one factor per (block, head): exp2(snapshot - M) (/ L when this workgroup saw the whole context), written
        // over the snapshot; entry e belongs to head e % G, whose M and L are folded again from the waves' values
        // (in the order used above).  The barrier inside the merge below publishes the factors
        for (int e = tid; e < max(te - tb, 0) * G; e += 64 * WAVES) {
            const int h = e % G;
            float Mh = -INFINITY;
#pragma unroll
            for (int w = 0; w < WAVES; ++w) Mh = fmaxf(Mh, wave_ml[(w * 16 + h) * 2]);
            float fl = 1.0f;
            if (final_out) {
                float Lh = 0.0f;
#pragma unroll
                for (int w = 0; w < WAVES; ++w) {
                    const float mw = wave_ml[(w * 16 + h) * 2];
                    Lh += (mw == -INFINITY) ? 0.0f : wave_ml[(w * 16 + h) * 2 + 1] * __builtin_amdgcn_exp2f(mw - Mh);
                }
                fl = Lh > 0.0f ? 1.0f / Lh : 0.0f;
            }
            msnap[e] = __builtin_amdgcn_exp2f(msnap[e] - Mh) * fl;
        }
    }
#pragma unroll
    for (int half = 0; half < 2; ++half) {
        if (half) __syncthreads();
#pragma unroll
        for (int r = 0; r < HALF; ++r)
#pragma unroll
            for (int i = 0; i < 4; ++i) red[((wv * HALF + r) * 4 + i) * 64 + lane] = acc[half * HALF + r][i] * f_own;
        __syncthreads();
        for (int r = wv; r < HALF; r += WAVES) {
            const int rr = half * HALF + r;
            float v[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                v[i] = 0.0f;
#pragma unroll
                for (int w = 0; w < WAVES; ++w) v[i] += red[((w * HALF + r) * 4 + i) * 64 + lane];
            }
            // lane (n, g), register i of tile rr holds channel 16 rr + 4 g + i of head n
            if (n < G) {
                if (final_out) {
                    uint16_t* o = a.out + ((long)t * Hq + hq) * D + 16 * rr + 4 * g;
                    *reinterpret_cast<uint2*>(o) = make_uint2(pack2<DT>(v[0] * inv_l, v[1] * inv_l), pack2<DT>(v[2] * inv_l, v[3] * inv_l));
                } else {
                    *reinterpret_cast<f4*>(a.part_acc + prow * D + 16 * rr + 4 * g) = f4{v[0], v[1], v[2], v[3]};
                }
            }
        }
    }
    if (wv == 0 && g == 0 && n < G) {
        float* ml = final_out ? a.final_ml + 2 * ((long)t * Hq + hq) : a.part_ml + 2 * prow;
        ml[0] = M;
        ml[1] = L;
    }

    // ---- scores: the factors were formed in place of the block maxima before the merge --------------
    if (!a.want_scores) return;
    const float* fac = msnap;
    typedef _Float16 h4 __attribute__((ext_vector_type(4)));
    typedef _Float16 h4u __attribute__((ext_vector_type(4), aligned(2)));
    const long soff = st.score_offsets[b];
    if (final_out) {
        // sum over the group's heads -> group_scores[hkv][position] (fp16, as in the u8 decode kernel), four positions
        // per thread; positions before the first block of the window get 0
        _Float16* dst = a.group_scores + (long)hkv * a.total_scores + soff;
        const int p0 = tb * TOK;
        for (int pos = tid; pos < p0; pos += 64 * WAVES) dst[pos] = (_Float16)0.0f;
        const int cnt = kv_len - p0;
        for (int lp = 4 * tid; lp < cnt; lp += 4 * 64 * WAVES) {
            const float* f = fac + (lp / TOK) * G;
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
            for (int pos = p_lo + 4 * tid; pos < p_hi; pos += 4 * 64 * WAVES) {
                const int lp = pos - p_lo;
                const float fh = fac[(lp / TOK) * G + h];
                const h4 p4 = *reinterpret_cast<const h4*>(ptile + h * pstride + lp);
                *reinterpret_cast<h4*>(dst + pos) = h4{(_Float16)((float)p4[0] * fh), (_Float16)((float)p4[1] * fh),
                                                       (_Float16)((float)p4[2] * fh), (_Float16)((float)p4[3] * fh)};
            }
        }
    }
}

template <int D, int DT, int BS>
hipError_t launch_decode16_sized(hipStream_t s, const DecodeArgs& a_in, hipEvent_t ev0, hipEvent_t ev1) {
    DecodeArgs a = a_in;
    size_t lds = decode16_lds_bytes(D, a.G, a.max_tiles, a.want_scores != 0);
    a.table_off = (int32_t)lds;
    lds += decode16_table_bytes(a.max_tiles, BS);
    auto kern = pa_decode16_kernel<D, DT, BS>;
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) return e;
    if (ev0) (void)hipEventRecord(ev0, s);
    hipLaunchKernelGGL(kern, dim3((unsigned)a.n_seqs * a.sh.Hkv * a.nsplit), dim3(256), lds, s, a);
    if (ev1) (void)hipEventRecord(ev1, s);
    return hipGetLastError();
}

template <int D, int DT>
hipError_t launch_decode16_typed(hipStream_t s, const DecodeArgs& a, hipEvent_t ev0, hipEvent_t ev1) {
    return a.sh.bs == 16 ? launch_decode16_sized<D, DT, 16>(s, a, ev0, ev1) : launch_decode16_sized<D, DT, 32>(s, a, ev0, ev1);
}

}  // namespace

size_t decode16_table_bytes(int max_tiles, int block_size) {
    return ((size_t)max_tiles * (block_size == 16 ? 2 : 1) * sizeof(int32_t) + 15) & ~(size_t)15;
}

// LDS in front of the block-table slice: V slots | per-wave (m, l) | [scores: block maxima | probabilities]
size_t decode16_lds_bytes(int D, int G, int max_tiles, bool want_scores) {
    size_t bytes = (size_t)4 * TOK * (D * 2 + 32) + 4 * 16 * 2 * sizeof(float);
    if (want_scores) bytes += (size_t)decode16_snap_floats(max_tiles, G) * sizeof(float) + (size_t)G * max_tiles * TOK * sizeof(uint16_t);
    return (bytes + 15) & ~(size_t)15;
}

hipError_t preload_decode16() {  // (see preload_decode_u8)
    hipFuncAttributes at;
    return hipFuncGetAttributes(&at, reinterpret_cast<const void*>(pa_decode16_kernel<128, DT_F16, 32>));
}

hipError_t launch_decode16(hipStream_t s, const DecodeArgs& a, int dtype, float* scores, int max_kv_len, hipEvent_t ev0,
                           hipEvent_t ev1) {
    if (a.sh.bs < 16 || a.sh.bs > 256 || (a.sh.bs & (a.sh.bs - 1)) || a.G > 16 || (a.want_scores != 0) != (scores != nullptr)) return hipErrorInvalidValue;
    hipError_t e;
    if (a.sh.D == 128) e = dtype == DT_F16 ? launch_decode16_typed<128, DT_F16>(s, a, ev0, ev1) : launch_decode16_typed<128, DT_BF16>(s, a, ev0, ev1);
    else if (a.sh.D == 64) e = dtype == DT_F16 ? launch_decode16_typed<64, DT_F16>(s, a, ev0, ev1) : launch_decode16_typed<64, DT_BF16>(s, a, ev0, ev1);
    else if (a.sh.D == 96) e = dtype == DT_F16 ? launch_decode16_typed<96, DT_F16>(s, a, ev0, ev1) : launch_decode16_typed<96, DT_BF16>(s, a, ev0, ev1);
    else if (a.sh.D == 256) e = dtype == DT_F16 ? launch_decode16_typed<256, DT_F16>(s, a, ev0, ev1) : launch_decode16_typed<256, DT_BF16>(s, a, ev0, ev1);
    else return hipErrorInvalidValue;
    if (e != hipSuccess) return e;
    return launch_decode_post(s, a, dtype, scores, max_kv_len);
}

}  // namespace pa
