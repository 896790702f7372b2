// Attention scores by replaying the last W query tokens of every sequence against the keys they see, on the
// gfx950 matrix cores.  Runs after the attention kernel, which leaves each query row's softmax maximum and
// denominator in `final_ml`:
//   score[pos] = sum over (heads, last W tokens i) of exp(scale * q_i . k_pos - M_row) / L_row   (masked entries 0)
// For a block-sparse sequence a row contributes only to the key blocks it kept (its maximum and denominator were
// formed over those).
//
// One wave owns 32 consecutive positions of one sequence; a workgroup is four such waves, nothing is shared
// between them (no LDS, no barriers).  Per kv head the wave loads its 32 key rows straight into MFMA B operands
// (lane (n, g): token 16 c + n, channels 32 s + 8 g .. + 7), then walks the W x G query rows of the head group in
// tiles of 16 as A operands:
//   S[row][token] = Q . K^T         v_mfma_f32_16x16x32_{f16,bf16}
// so that lane (n, g) receives rows 4 g + i of token column n: the sum over rows is in-lane adds plus two
// cross-lane steps at the very end, and all kv heads accumulate in registers -- every score is written once,
// by one lane, in a fixed order (no atomics).
// u8 caches: codes become f16 operands by zero extension (the subnormal code * 2^-24, multiplied exactly) and the
// row's scale / zero-point are applied to the accumulator:  logit = scale * sc_k * (q . codes - zp_k * sum(q)).
//
// Roofline: HBM for W = 1 (the K rows are read once, 32 x row bytes per wave and kv head); dense MFMA for wide
// windows (2 * D flops per (row, position)).
#include "pa_device.h"

namespace pa {
namespace {

typedef _Float16 h8 __attribute__((ext_vector_type(8)));
typedef __bf16 b8 __attribute__((ext_vector_type(8)));
typedef short s8v __attribute__((ext_vector_type(8)));
typedef float f4 __attribute__((ext_vector_type(4)));
typedef uint32_t u4v __attribute__((ext_vector_type(4)));

constexpr float LOG2E = 1.4426950408889634f;
constexpr int TN = 32;  // positions per wave
constexpr int CG = TN / 16;

template <int DT>
__device__ __forceinline__ f4 mma(const s8v& a, const s8v& b, const f4& c) {
    if (DT == DT_F16)
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(h8, a), __builtin_bit_cast(h8, b), c, 0, 0, 0);
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(b8, a), __builtin_bit_cast(b8, b), c, 0, 0, 0);
}

__device__ __forceinline__ uint32_t f16x2(float a, float b) {
    typedef _Float16 h2 __attribute__((ext_vector_type(2)));
    return __builtin_bit_cast(uint32_t, h2{(_Float16)a, (_Float16)b});
}

__device__ __forceinline__ float sum_over_g(float v) {
    v += __shfl_xor(v, 16, WAVE);
    return v + __shfl_xor(v, 32, WAVE);
}

// DT: MFMA operand type; QDT: type of the query; U8: `f32 scale | f32 zero-point | D codes` key rows.
template <int D, int DT, int QDT, bool U8>
__global__ __launch_bounds__(256) void pa_scores_mfma_kernel(StepDev st, Shape sh, const uint16_t* __restrict__ query,
                                                             const uint8_t* __restrict__ key_cache,
                                                             const int32_t* __restrict__ block_indices,
                                                             const float* __restrict__ final_ml,
                                                             float* __restrict__ scores,
                                                             const int32_t* __restrict__ seq_list, int n_seqs,
                                                             XattDev xd, SingleScores ss, MergeRows mg) {
    static_assert(!U8 || DT == DT_F16, "u8 codes are multiplied as f16");
    constexpr int KS = D / 32;
    constexpr int CROWB = U8 ? D + 8 : D * 2;
    constexpr float CODE_UNIT = 16777216.0f;  // a code byte read as f16 is code * 2^-24
    if ((int)blockIdx.y >= n_seqs + ss.n_seqs) {  // the last rows: the fold of the matrix kernel's partial rows
        const long wg = (long)((int)blockIdx.y - n_seqs - ss.n_seqs) * gridDim.x + blockIdx.x;
        if (wg < mg.n_wg) merge_rows<D, QDT>(mg, wg);
        return;
    }
    if ((int)blockIdx.y >= n_seqs) {  // the rows behind the sequences': single-token sequences whose probabilities were kept
        single_scores_rows(st, sh, ss, final_ml, mg, scores, (int)blockIdx.y - n_seqs, (int)blockIdx.x);
        return;
    }
    const int b = seq_list ? seq_list[blockIdx.y] : (int)blockIdx.y;  // the listed sequences, or all of the step's
    const int t0 = st.subsequence_begins[b];
    const int q_len = st.subsequence_begins[b + 1] - t0;
    const int past = st.past_lens[b];
    const int kv_len = past + q_len;
    const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
    const int n = lane & 15, g = lane >> 4;
    const int base = (blockIdx.x * 4 + wv) * TN;
    if (base >= kv_len) return;
    const int W = st.score_window[b];
    const int Hq = sh.Hq, Hkv = sh.Hkv, G = Hq / Hkv;
    const int bs_shift = 31 - __builtin_clz(sh.bs);  // cache blocks of 16 to 256 tokens (a power of two)
    const int R = W * G;                       // query rows per kv head
    const int first_tok = t0 + q_len - W;      // first of the last W tokens
    const int first_pos = past + q_len - W;    // its position
    const int sw = st.sliding_window;
    const int lo_any = sw > 0 ? max(0, first_pos + 1 - sw) : 0;  // below this no row sees anything
    const int32_t* table = block_indices + st.block_indices_begins[b];
    const float scl = st.scale * LOG2E;
    const float inv_g = 1.0f / (float)G;
    const int xi = xd.seq_of ? xd.seq_of[b] : -1;  // block-sparse sequence: the wave's 32 positions lie in one key block

    // Rows cut into ranges, one query token, at most 64 heads (the usual case): lane h folds head h's maximum and
    // denominator once, up front, and the row loop below fetches them from that lane.
    const bool lane_rows = mg.n_merge > 0 && W == 1 && Hq <= WAVE;
    float2 ml_lane = make_float2(0.0f, 0.0f);
    if (lane_rows) ml_lane = row_max_and_sum_wide(final_ml, mg, first_tok, (long)first_tok * Hq + min(lane, Hq - 1));

    float total[CG];
#pragma unroll
    for (int c = 0; c < CG; ++c) total[c] = 0.0f;

    if (W > 0 && base + TN > lo_any) {
        for (int hkv = 0; hkv < Hkv; ++hkv) {
            // ---- this wave's 64 key rows of the kv head, as B operands ------------------------------
            s8v kreg[CG][KS];
            float sck[CG], zpk[CG];  // u8: scale * scl * 2^24 and zero-point * scale * scl of the lane's token
#pragma unroll
            for (int c = 0; c < CG; ++c) {
                // positions beyond the sequence repeat its last row: no branch around the loads, so that they all go
                // out back to back (behind a branch each load was waited for before the next was issued); such
                // columns are masked below, where every row's limit is below kv_len
                const int pos = min(base + 16 * c + n, kv_len - 1);
                const uint8_t* row = key_cache + (((long)table[pos >> bs_shift] * Hkv + hkv) * sh.bs + (pos & (sh.bs - 1))) * CROWB;
                if (U8) {
                    const float2 hd = *reinterpret_cast<const float2*>(row);
                    sck[c] = hd.x * scl * CODE_UNIT;
                    zpk[c] = hd.y * hd.x * scl;
                }
#pragma unroll
                for (int s = 0; s < KS; ++s) {
                    u4v v;
                    if (U8) {
                        typedef uint32_t u2v __attribute__((ext_vector_type(2)));
                        const u2v cd = *reinterpret_cast<const u2v*>(row + 8 + 32 * s + 8 * g);
                        v = u4v{__builtin_amdgcn_perm(0u, cd[0], 0x0c010c00u), __builtin_amdgcn_perm(0u, cd[0], 0x0c030c02u),
                                __builtin_amdgcn_perm(0u, cd[1], 0x0c010c00u), __builtin_amdgcn_perm(0u, cd[1], 0x0c030c02u)};
                    } else {
                        v = *reinterpret_cast<const u4v*>(row + (32 * s + 8 * g) * 2);
                    }
                    kreg[c][s] = __builtin_bit_cast(s8v, v);
                }
            }
            // ---- the head group's W x G query rows, 16 at a time --------------------------------------
            for (int r0 = 0; r0 < R; r0 += 16) {
                // A operand: row r0 + n = (token (r0 + n) / G of the window, head (r0 + n) % G of the group)
                s8v qreg[KS];
                float qsum_a = 0.0f;
                {
                    const int row = min(r0 + n, R - 1);  // rows beyond R repeat the last one; they are masked below
                    const int tok = (int)(((float)row + 0.5f) * inv_g);
                    const uint16_t* q = query + ((long)(first_tok + tok) * Hq + hkv * G + (row - tok * G)) * D;
#pragma unroll
                    for (int s = 0; s < KS; ++s) {
                        u4v v = *reinterpret_cast<const u4v*>(q + 32 * s + 8 * g);
                        if (QDT != DT) {  // bf16 query against f16 operands
#pragma unroll
                            for (int e = 0; e < 4; ++e)
                                v[e] = f16x2(__builtin_bit_cast(float, v[e] << 16), __builtin_bit_cast(float, v[e] & 0xffff0000u));
                        }
                        qreg[s] = __builtin_bit_cast(s8v, v);
                        if (U8) {
                            const h8 qh = __builtin_bit_cast(h8, v);
#pragma unroll
                            for (int e = 0; e < 8; ++e) qsum_a += (float)qh[e];
                        }
                    }
                    if (U8) qsum_a = sum_over_g(qsum_a);
                }
                // accumulator rows of this lane: r0 + 4 g + i
                float m2[4], inv_l[4], qs[4];
                int rpos[4];
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const bool ok = r0 + 4 * g + i < R;
                    const int row = min(r0 + 4 * g + i, R - 1);
                    const int tok = (int)(((float)row + 0.5f) * inv_g);
                    const long rid = (long)(first_tok + tok) * Hq + hkv * G + (row - tok * G);
                    float2 ml;
                    if (lane_rows) {
                        const int head = hkv * G + (row - tok * G);
                        ml = make_float2(__shfl(ml_lane.x, head, WAVE), __shfl(ml_lane.y, head, WAVE));
                    } else {
                        ml = row_max_and_sum(final_ml, mg, first_tok + tok, rid);
                    }
                    m2[i] = ml.x * LOG2E;
                    inv_l[i] = ml.y > 0.0f ? 1.0f / ml.y : 0.0f;
                    rpos[i] = ok ? first_pos + tok : -1;  // -1: sees nothing
                    if (xi >= 0) {
                        const XattSeq xs = xd.seqs[xi];
                        const int J = base >> xd.xb_shift;
                        const int I = min((first_pos + tok) >> xd.xb_shift, xs.nkb - 1);
                        const uint32_t* mrow = xd.mask + xs.mask_off +
                                               ((long)(hkv * G + (row - tok * G)) * xs.nqb + (I - xs.qb0)) * xs.words;
                        if (J > I || !((mrow[J >> 5] >> (J & 31)) & 1u)) rpos[i] = -1;
                    }
                    qs[i] = U8 ? __shfl(qsum_a, 4 * g + i, WAVE) : 0.0f;
                }
#pragma unroll
                for (int c = 0; c < CG; ++c) {
                    f4 acc = f4{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
                    for (int s = 0; s < KS; ++s) acc = mma<DT>(qreg[s], kreg[c][s], acc);
                    const int pos = base + 16 * c + n;
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        const float x = U8 ? fmaf(acc[i], sck[c], -zpk[c] * qs[i]) : acc[i] * scl;
                        const int low = sw > 0 ? rpos[i] + 1 - sw : 0;
                        const float p = __builtin_amdgcn_exp2f(x - m2[i]) * inv_l[i];
                        total[c] += (pos <= rpos[i] && pos >= low) ? p : 0.0f;
                    }
                }
            }
        }
    }
    float* out = scores + st.score_offsets[b];
#pragma unroll
    for (int c = 0; c < CG; ++c) {
        const float v = sum_over_g(total[c]);
        const int pos = base + 16 * c + n;
        if (g == 0 && pos < kv_len) out[pos] = v;
    }
}

}  // namespace

hipError_t launch_scores_replay(hipStream_t s, const StepDev& st, const Shape& sh, int q_dtype, int kv_dtype,
                                const void* query, const void* key_cache, const int32_t* block_indices,
                                float* final_ml, float* scores, int32_t max_kv_len, const int32_t* seq_list,
                                int32_t n_seqs, const XattDev& xd, const SingleScores& ss_in, const MergeRows& mg_in) {
    SingleScores ss = ss_in;
    if (!ss.p_out) ss.n_seqs = 0;
    MergeRows mg = mg_in;
    if (mg.n_merge <= 0) mg.n_wg = 0;
    if (max_kv_len <= 0 || (n_seqs + ss.n_seqs == 0 && mg.n_wg == 0)) return mg.n_wg ? hipErrorInvalidValue : hipSuccess;
    const int gx_all = ceil_div(max_kv_len, 4 * TN);
    const int merge_rows_y = ceil_div(mg.n_wg, gx_all);
    if (sh.Hq > 256 || n_seqs + ss.n_seqs + merge_rows_y > 65535) return hipErrorInvalidValue;
    const dim3 grid((unsigned)gx_all, (unsigned)(n_seqs + ss.n_seqs + merge_rows_y)), block(256);
    ss.gx = min(ceil_div(max_kv_len, 2048), 64);  // (at most the grid's width: 2048 > 4 * TN)
    auto q = reinterpret_cast<const uint16_t*>(query);
    auto k = reinterpret_cast<const uint8_t*>(key_cache);
#define PA_REPLAY(DD, DT, Q, U8)                                                                               \
    {                                                                                                          \
        hipLaunchKernelGGL((pa_scores_mfma_kernel<DD, DT, Q, U8>), grid, block, 0, s, st, sh, q, k,            \
                           block_indices, final_ml, scores, seq_list, n_seqs, xd, ss, mg);                     \
        return hipGetLastError();                                                                              \
    }
    if (sh.bs < 16 || sh.bs > 256 || (sh.bs & (sh.bs - 1))) return hipErrorInvalidValue;
    if (kv_dtype == DT_U8) {
        if (sh.D == 64 && q_dtype == DT_F16) PA_REPLAY(64, DT_F16, DT_F16, true)
        if (sh.D == 64 && q_dtype == DT_BF16) PA_REPLAY(64, DT_F16, DT_BF16, true)
        if (sh.D == 128 && q_dtype == DT_F16) PA_REPLAY(128, DT_F16, DT_F16, true)
        if (sh.D == 128 && q_dtype == DT_BF16) PA_REPLAY(128, DT_F16, DT_BF16, true)
        if (sh.D == 96 && q_dtype == DT_F16) PA_REPLAY(96, DT_F16, DT_F16, true)
        if (sh.D == 96 && q_dtype == DT_BF16) PA_REPLAY(96, DT_F16, DT_BF16, true)
        if (sh.D == 256 && q_dtype == DT_F16) PA_REPLAY(256, DT_F16, DT_F16, true)
        if (sh.D == 256 && q_dtype == DT_BF16) PA_REPLAY(256, DT_F16, DT_BF16, true)
    } else if (kv_dtype == q_dtype) {
        if (sh.D == 64 && q_dtype == DT_F16) PA_REPLAY(64, DT_F16, DT_F16, false)
        if (sh.D == 64 && q_dtype == DT_BF16) PA_REPLAY(64, DT_BF16, DT_BF16, false)
        if (sh.D == 128 && q_dtype == DT_F16) PA_REPLAY(128, DT_F16, DT_F16, false)
        if (sh.D == 128 && q_dtype == DT_BF16) PA_REPLAY(128, DT_BF16, DT_BF16, false)
        if (sh.D == 96 && q_dtype == DT_F16) PA_REPLAY(96, DT_F16, DT_F16, false)
        if (sh.D == 96 && q_dtype == DT_BF16) PA_REPLAY(96, DT_BF16, DT_BF16, false)
        if (sh.D == 256 && q_dtype == DT_F16) PA_REPLAY(256, DT_F16, DT_F16, false)
        if (sh.D == 256 && q_dtype == DT_BF16) PA_REPLAY(256, DT_BF16, DT_BF16, false)
    }
#undef PA_REPLAY
    return hipErrorInvalidValue;
}

}  // namespace pa
