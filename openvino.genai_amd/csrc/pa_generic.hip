// Shape-generic PagedAttention kernels: any block size and GQA ratio, q_len >= 1, key and value head sizes that are
// multiples of 8 up to 512 and need not be equal, and an element type per cache tensor -- f16, bf16, u8 rows
// (`f32 scale | f32 zero-point | D codes`) or u4 rows (`f32 scale | f32 zero-point | D / 2 bytes`, element 2 i in the
// high nibble of byte i).  Everything the tuned kernels do not take runs here.
//
// pa_generic_kernel     : one wave per (tile of consecutive tokens of a sequence, kv head, heads of its group, split): up
//                         to eight query rows.  Lanes take consecutive KV positions for QK (each lane owns one cache
//                         row, read once for all the rows), then regroup across the value head for PV.  Online softmax
//                         per query row and wave.
// pa_merge_kernel       : folds the split partials (m, l, acc) into the output row and keeps the final
//                         (max, denominator) of every (token, head) for the score kernels.
// pa_scores_single      : scores of single-token (decode) sequences from the stored logits.
// pa_scores_window      : scores of multi-token sequences: recomputes QK for the last W query rows.
// kv_append_generic     : one wave per (token, kv head, K | V) row: copy / convert / quantise into the cache row.
//
// HBM-bound, no MFMA: a fallback, not a tuned path.
#include "pa_device.h"

namespace pa {
namespace {

constexpr int MAX_D = GENERIC_MAX_HEAD_SIZE;

// One cached row of D elements in the tensor's element type, read as f32.
struct RowReader {
    const uint8_t* row;
    float scale, zp;
    int dt;
    __device__ RowReader(const uint8_t* cache, long phys, int h, int slot, int Hkv, int bs, int D, int dt_) : dt(dt_) {
        row = cache + ((phys * Hkv + h) * bs + slot) * (long)row_bytes(D, dt_);
        scale = 1.0f;
        zp = 0.0f;
        if (dt == DT_U8 || dt == DT_U4) {
            const float2 hdr = *reinterpret_cast<const float2*>(row);
            scale = hdr.x;
            zp = hdr.y;
            row += 8;
        }
    }
    // eight consecutive elements starting at d (d % 8 == 0)
    __device__ void load8(int d, float* out) const {
        if (dt == DT_U8) {
            const uint2 v = *reinterpret_cast<const uint2*>(row + d);
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                out[e] = ((float)((v.x >> (8 * e)) & 0xff) - zp) * scale;
                out[4 + e] = ((float)((v.y >> (8 * e)) & 0xff) - zp) * scale;
            }
        } else if (dt == DT_U4) {
            const uint32_t v = *reinterpret_cast<const uint32_t*>(row + d / 2);
#pragma unroll
            for (int e = 0; e < 4; ++e) {  // byte e holds elements 2 e (high nibble) and 2 e + 1 (low nibble)
                const uint32_t byte = (v >> (8 * e)) & 0xff;
                out[2 * e] = ((float)(byte >> 4) - zp) * scale;
                out[2 * e + 1] = ((float)(byte & 15) - zp) * scale;
            }
        } else {
            const uint4 v = *reinterpret_cast<const uint4*>(row + 2 * d);
            const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                out[2 * e] = dt == DT_F16 ? half_bits_to_float((uint16_t)(w[e] & 0xffff)) : bf16_bits_to_float((uint16_t)(w[e] & 0xffff));
                out[2 * e + 1] = dt == DT_F16 ? half_bits_to_float((uint16_t)(w[e] >> 16)) : bf16_bits_to_float((uint16_t)(w[e] >> 16));
            }
        }
    }
    // eight consecutive elements as stored: the codes of u8 / u4 rows (the element is (code - zp) * scale), the values
    // of 16-bit rows (scale 1, zero-point 0)
    __device__ void load8_codes(int d, float* out) const {
        if (dt == DT_U8) {
            const uint2 v = *reinterpret_cast<const uint2*>(row + d);
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                out[e] = (float)((v.x >> (8 * e)) & 0xff);
                out[4 + e] = (float)((v.y >> (8 * e)) & 0xff);
            }
        } else if (dt == DT_U4) {
            const uint32_t v = *reinterpret_cast<const uint32_t*>(row + d / 2);
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const uint32_t byte = (v >> (8 * e)) & 0xff;
                out[2 * e] = (float)(byte >> 4);
                out[2 * e + 1] = (float)(byte & 15);
            }
        } else {
            load8(d, out);
        }
    }
    __device__ float load1(int d) const {
        if (dt == DT_U8) return ((float)row[d] - zp) * scale;
        if (dt == DT_U4) {
            const uint8_t byte = row[d >> 1];
            return ((float)((d & 1) ? (byte & 15) : (byte >> 4)) - zp) * scale;
        }
        const uint16_t v = reinterpret_cast<const uint16_t*>(row)[d];
        return dt == DT_F16 ? half_bits_to_float(v) : bf16_bits_to_float(v);
    }
};

// One wave per (token tile, kv head, set of heads of its group, split): GC query rows -- `hs` heads for each of the
// tile's GC / hs consecutive tokens of one sequence -- share every cache row the wave touches.  QK: a lane owns a
// position, walks its key row eight elements at a time against the query rows (scaled, f32, in LDS: all lanes read the
// same words); each row masks what its token may not see.  PV: the lanes regroup -- LPR lanes to a value row, eight
// channels each, 64 / LPR rows per step -- and fetch the rows' probabilities from the lanes that own them; the row
// groups' partial sums are added once at the end.  Online softmax per query row and wave.
template <int QDT, int GC>
__global__ __launch_bounds__(256, GC <= 4 ? 4 : 2) void pa_generic_kernel(StepDev st, GenericShape sh, const uint16_t* __restrict__ query,
                                                         const uint8_t* __restrict__ key_cache,
                                                         const uint8_t* __restrict__ value_cache,
                                                         const int32_t* __restrict__ block_indices, AttnWorkspace ws,
                                                         int store_logits, int hs) {
    extern __shared__ float qs_all[];  // [4 waves][GC][Dk]
    const int lane = threadIdx.x & 63;
    const int wv = threadIdx.x >> 6;
    const int Dk = sh.Dk, Dv = sh.Dv;
    const int G = sh.Hq / sh.Hkv;
    const int sets = ceil_div(G, hs);
    const long wave = (long)blockIdx.x * 4 + wv;
    const long total = (long)st.n_gtiles * sh.Hkv * sets * ws.nsplit;
    const bool valid = wave < total;
    float* qs = qs_all + (long)wv * GC * Dk;
    int split = 0, hkv = 0, t0 = 0, nt = 0, g0 = 0, ng = 0;
    if (valid) {
        split = (int)(wave % ws.nsplit);
        const int set = (int)((wave / ws.nsplit) % sets);
        hkv = (int)((wave / ((long)ws.nsplit * sets)) % sh.Hkv);
        const int tile = st.gtiles[wave / ((long)ws.nsplit * sets * sh.Hkv)];
        t0 = tile >> 3;          // the tile's first token
        nt = (tile & 7) + 1;     // its tokens
        g0 = set * hs;
        ng = min(hs, G - g0);
        // row r = (token t0 + r / hs, head g0 + r % hs); rows beyond the tile or the group are zero and write nothing
        for (int idx = lane; idx < GC * Dk; idx += 64) {
            const int r = idx / Dk, d = idx - r * Dk;
            const int ti = r / hs, g = r - ti * hs;
            qs[idx] = (ti < nt && g < ng) ? load16<QDT>(query[((long)(t0 + ti) * sh.Hq + hkv * G + g0 + g) * Dk + d]) * st.scale : 0.0f;
        }
    }
    __syncthreads();
    if (!valid) return;
    // Quantised rows are multiplied as codes; scale and zero-point come in once per row:
    //   q . k = scale_k (q . codes - zp_k sum(q)),   sum_j p_j v_j = sum_j (p_j scale_v) codes_j - sum_j p_j scale_v zp_v
    float qsum[GC];
#pragma unroll
    for (int r = 0; r < GC; ++r) {
        float part = 0.0f;
        for (int d = lane; d < Dk; d += 64) part += qs[r * Dk + d];
        qsum[r] = __builtin_bit_cast(float, __builtin_amdgcn_readfirstlane(__builtin_bit_cast(int, wave_sum(part))));  // (the same in every lane)
    }

    const int b = st.token_seq[t0];
    const int i0 = t0 - st.subsequence_begins[b];
    const int q_len = st.subsequence_begins[b + 1] - st.subsequence_begins[b];
    const int past = st.past_lens[b];
    const int sw = st.sliding_window;
    // what the tile's tokens see together: from the first token's first position to the last token's own
    const int last_w = past + i0 + nt - 1;
    const int first_w = sw > 0 ? max(0, past + i0 + 1 - sw) : 0;
    const int n = last_w + 1 - first_w;
    const int chunk = ceil_div(ceil_div(n, ws.nsplit), 64) * 64;
    const int j_begin = first_w + split * chunk;
    const int j_end = min(last_w + 1, j_begin + chunk);
    const int32_t* table = block_indices + st.block_indices_begins[b];
    const bool keep_logits = store_logits && q_len == 1 && st.score_window[b] > 0;
    const int hq0 = hkv * G + g0;
    float slope[GC];
    int row_last[GC], row_first[GC];  // the positions row r sees: [row_first, row_last]; none for rows that do not exist
#pragma unroll
    for (int r = 0; r < GC; ++r) {
        const int ti = r / hs, g = r - ti * hs;
        const bool exists = ti < nt && g < ng;
        slope[r] = ws.alibi && exists ? ws.alibi[hq0 + g] : 0.0f;
        row_last[r] = exists ? past + i0 + ti : -1;
        row_first[r] = sw > 0 ? max(0, past + i0 + ti + 1 - sw) : 0;
    }

    // value rows: LPR lanes to a row (a power of two, at least Dv / 8), RPS rows per step
    int lpr = 1;
    while (lpr * 8 < Dv) lpr <<= 1;
    const int rps = 64 / lpr;
    const int vlane = lane & (lpr - 1), vrow = lane / lpr;
    const bool v_active = 8 * vlane < Dv;

    float m[GC], l[GC], acc[GC][8], zacc[GC];
#pragma unroll
    for (int r = 0; r < GC; ++r) {
        m[r] = -INFINITY;
        l[r] = 0.0f;
        zacc[r] = 0.0f;
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[r][e] = 0.0f;
    }

    for (int j0 = j_begin; j0 < j_end; j0 += 64) {
        const int j = j0 + lane;
        const bool live = j < j_end;
        long phys = 0;
        float sc[GC];
#pragma unroll
        for (int r = 0; r < GC; ++r) sc[r] = 0.0f;
        if (live) {
            phys = table[j / sh.bs];
            RowReader kr(key_cache, phys, hkv, j % sh.bs, sh.Hkv, sh.bs, Dk, sh.kdt);
            for (int d = 0; d < Dk; d += 8) {
                float k8[8];
                kr.load8_codes(d, k8);
#pragma unroll
                for (int r = 0; r < GC; ++r) {
                    const float* qr = qs + r * Dk + d;
#pragma unroll
                    for (int e = 0; e < 8; ++e) sc[r] += qr[e] * k8[e];
                }
            }
#pragma unroll
            for (int r = 0; r < GC; ++r) sc[r] = kr.scale * (sc[r] - kr.zp * qsum[r]);
        }
        float p[GC];
#pragma unroll
        for (int r = 0; r < GC; ++r) {
            float x = -INFINITY;
            if (live && j <= row_last[r] && j >= row_first[r]) {
                x = ws.alibi ? sc[r] + slope[r] * (float)(j - row_last[r]) : sc[r];
                if (keep_logits) ws.logits[(long)(hq0 + r) * ws.total_scores + st.score_offsets[b] + j] = x;  // (one token: r = head)
            }
            const float m_new = fmaxf(m[r], wave_max(x));
            const float corr = (m[r] == -INFINITY) ? 0.0f : __expf(m[r] - m_new);
            p[r] = x == -INFINITY ? 0.0f : __expf(x - m_new);  // (a row that has seen nothing yet: m_new = -inf too)
            l[r] = l[r] * corr + wave_sum(p[r]);
#pragma unroll
            for (int e = 0; e < 8; ++e) acc[r][e] *= corr;
            zacc[r] *= corr;
            m[r] = m_new;
        }
        const int cnt = min(64, j_end - j0);
        for (int s = 0; s * rps < cnt; ++s) {
            const int jj = s * rps + vrow;            // the row of this lane's group in this step
            const int src = min(jj, 63);
            const long pb = __shfl(phys, src, WAVE);
            float pj[GC];
#pragma unroll
            for (int r = 0; r < GC; ++r) pj[r] = __shfl(p[r], src, WAVE);
            if (v_active && jj < cnt) {
                RowReader vr(value_cache, pb, hkv, (j0 + jj) % sh.bs, sh.Hkv, sh.bs, Dv, sh.vdt);
                float v8[8];
                vr.load8_codes(8 * vlane, v8);
#pragma unroll
                for (int r = 0; r < GC; ++r) {
                    const float w = pj[r] * vr.scale;
                    zacc[r] += w * vr.zp;
#pragma unroll
                    for (int e = 0; e < 8; ++e) acc[r][e] += w * v8[e];
                }
            }
        }
    }
    // the zero-point terms of the lane's rows, then the row groups' partial sums: lanes with the same channels add up
#pragma unroll
    for (int r = 0; r < GC; ++r)
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            acc[r][e] -= zacc[r];
            for (int o = lpr; o < 64; o <<= 1) acc[r][e] += __shfl_xor(acc[r][e], o, WAVE);
        }
#pragma unroll
    for (int r = 0; r < GC; ++r) {
        if (row_last[r] < 0) continue;
        const int ti = r / hs, g = r - ti * hs;
        const long slot = ((long)(t0 + ti) * sh.Hq + hq0 + g) * ws.nsplit + split;
        if (lane == 0) {
            ws.part_ml[2 * slot] = m[r];
            ws.part_ml[2 * slot + 1] = l[r];
        }
        if (vrow == 0 && v_active) {
            float* dst = ws.part_acc + slot * Dv + 8 * vlane;
#pragma unroll
            for (int e = 0; e < 8; ++e) dst[e] = acc[r][e];
        }
    }
}

template <int QDT>
__global__ __launch_bounds__(256) void pa_merge_kernel(StepDev st, GenericShape sh, AttnWorkspace ws, uint16_t* __restrict__ out) {
    constexpr int EPL = MAX_D / 64;
    const int lane = threadIdx.x & 63;
    const int Dv = sh.Dv;
    const long row = (long)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= (long)st.T * sh.Hq) return;
    float M = -INFINITY;
    for (int s = 0; s < ws.nsplit; ++s) M = fmaxf(M, ws.part_ml[2 * (row * ws.nsplit + s)]);
    float L = 0.0f;
    float acc[EPL];
#pragma unroll
    for (int e = 0; e < EPL; ++e) acc[e] = 0.0f;
    for (int s = 0; s < ws.nsplit; ++s) {
        const long slot = row * ws.nsplit + s;
        const float ms = ws.part_ml[2 * slot];
        if (ms == -INFINITY) continue;
        const float f = __expf(ms - M);
        L += ws.part_ml[2 * slot + 1] * f;
#pragma unroll
        for (int e = 0; e < EPL; ++e)
            if (lane + 64 * e < Dv) acc[e] += ws.part_acc[slot * Dv + lane + 64 * e] * f;
    }
    const float inv = L > 0.0f ? 1.0f / L : 0.0f;
#pragma unroll
    for (int e = 0; e < EPL; ++e)
        if (lane + 64 * e < Dv) out[row * Dv + lane + 64 * e] = store16<QDT>(acc[e] * inv);
    if (lane == 0) {
        ws.final_ml[2 * row] = M;
        ws.final_ml[2 * row + 1] = L;
    }
}

// Single-token sequences: score_j = sum over heads of exp(logit - M) / L, heads in ascending order.
__global__ __launch_bounds__(256) void pa_scores_single_kernel(StepDev st, GenericShape sh, AttnWorkspace ws,
                                                               float* __restrict__ scores) {
    const int b = blockIdx.y;
    const int q_len = st.subsequence_begins[b + 1] - st.subsequence_begins[b];
    if (q_len != 1) return;
    const int t = st.subsequence_begins[b];
    const int kv_len = st.past_lens[b] + 1;
    const int first = st.sliding_window > 0 ? max(0, kv_len - st.sliding_window) : 0;
    const int W = st.score_window[b];
    for (int j = blockIdx.x * 256 + threadIdx.x; j < kv_len; j += gridDim.x * 256) {
        float sum = 0.0f;
        if (W > 0 && j >= first) {
            for (int h = 0; h < sh.Hq; ++h) {
                const float M = ws.final_ml[2 * ((long)t * sh.Hq + h)];
                const float L = ws.final_ml[2 * ((long)t * sh.Hq + h) + 1];
                sum += __expf(ws.logits[(long)h * ws.total_scores + st.score_offsets[b] + j] - M) / L;
            }
        }
        scores[st.score_offsets[b] + j] = sum;
    }
}

// Multi-token sequences: the last W query rows are replayed against every position they can see.
template <int QDT>
__global__ __launch_bounds__(256) void pa_scores_window_kernel(StepDev st, GenericShape sh, AttnWorkspace ws,
                                                               const uint16_t* __restrict__ query,
                                                               const uint8_t* __restrict__ key_cache,
                                                               const int32_t* __restrict__ block_indices,
                                                               float* __restrict__ scores, int single_too) {
    const int b = blockIdx.y;
    const int t0 = st.subsequence_begins[b];
    const int q_len = st.subsequence_begins[b + 1] - t0;
    if (q_len <= 1 && !single_too) return;
    const int past = st.past_lens[b];
    const int kv_len = past + q_len;
    const int W = st.score_window[b];
    const int G = sh.Hq / sh.Hkv;
    const int Dk = sh.Dk;
    const int32_t* table = block_indices + st.block_indices_begins[b];
    for (int j = blockIdx.x * 256 + threadIdx.x; j < kv_len; j += gridDim.x * 256) {
        float sum = 0.0f;
        for (int i = q_len - W; i < q_len; ++i) {
            const int last = past + i;
            const int first = st.sliding_window > 0 ? max(0, last + 1 - st.sliding_window) : 0;
            if (j < first || j > last) continue;
            for (int h = 0; h < sh.Hq; ++h) {
                RowReader kr(key_cache, table[j / sh.bs], h / G, j % sh.bs, sh.Hkv, sh.bs, Dk, sh.kdt);
                const uint16_t* q = query + ((long)(t0 + i) * sh.Hq + h) * Dk;
                float dot = 0.0f;
                for (int d = 0; d < Dk; d += 8) {
                    float k8[8];
                    kr.load8(d, k8);
                    const uint4 qv = *reinterpret_cast<const uint4*>(q + d);
                    const uint32_t w[4] = {qv.x, qv.y, qv.z, qv.w};
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        dot += load16<QDT>((uint16_t)(w[e] & 0xffff)) * st.scale * k8[2 * e];
                        dot += load16<QDT>((uint16_t)(w[e] >> 16)) * st.scale * k8[2 * e + 1];
                    }
                }
                if (ws.alibi) dot += ws.alibi[h] * (float)(j - last);
                const float M = ws.final_ml[2 * ((long)(t0 + i) * sh.Hq + h)];
                const float L = ws.final_ml[2 * ((long)(t0 + i) * sh.Hq + h) + 1];
                sum += __expf(dot - M) / L;
            }
        }
        scores[st.score_offsets[b] + j] = sum;
    }
}

// One wave per (token, kv head, K | V) row.  u8 / u4 rows: scale = (max - min) / levels (a zero range takes 1e-4),
// zp = -min / scale, code = clamp(rne(fma(x, 1 / scale, zp)), 0, levels), every operation in IEEE binary32 without
// contraction, so that the bytes are reproducible on any IEEE host.  16-bit rows are copied, or converted when the cache
// holds the other 16-bit type.
template <int QDT>
__global__ __launch_bounds__(256) void kv_append_generic_kernel(StepDev st, GenericShape sh, const uint16_t* __restrict__ key,
                                                                const uint16_t* __restrict__ value,
                                                                uint8_t* __restrict__ key_cache,
                                                                uint8_t* __restrict__ value_cache,
                                                                const int32_t* __restrict__ block_indices) {
#pragma clang fp contract(off)
    const int lane = threadIdx.x & 63;
    const long row = (long)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= (long)st.T * sh.Hkv * 2) return;
    const int which = (int)(row & 1);
    const int h = (int)((row >> 1) % sh.Hkv);
    const int t = (int)((row >> 1) / sh.Hkv);
    const int D = which ? sh.Dv : sh.Dk, dt = which ? sh.vdt : sh.kdt;
    const int b = st.token_seq[t];
    const int slot = st.past_lens[b] + t - st.subsequence_begins[b];
    const long phys = block_indices[st.block_indices_begins[b] + slot / sh.bs];
    const uint16_t* src = (which ? value : key) + ((long)t * sh.Hkv + h) * D;
    uint8_t* dst = (which ? value_cache : key_cache) + ((phys * sh.Hkv + h) * sh.bs + slot % sh.bs) * (long)row_bytes(D, dt);
    constexpr int PPL = MAX_D / 128;  // element pairs per lane at most
    float x0[PPL], x1[PPL];
    float mn = INFINITY, mx = -INFINITY;
#pragma unroll
    for (int i = 0; i < PPL; ++i) {
        const int p = lane + 64 * i;
        if (2 * p < D) {
            const uint32_t w = reinterpret_cast<const uint32_t*>(src)[p];
            x0[i] = load16<QDT>((uint16_t)(w & 0xffff));
            x1[i] = load16<QDT>((uint16_t)(w >> 16));
            mn = fminf(mn, fminf(x0[i], x1[i]));
            mx = fmaxf(mx, fmaxf(x0[i], x1[i]));
        }
    }
    if (dt == DT_F16 || dt == DT_BF16) {
#pragma unroll
        for (int i = 0; i < PPL; ++i) {
            const int p = lane + 64 * i;
            if (2 * p < D) {
                const uint32_t lo = dt == DT_F16 ? float_to_half_bits(x0[i]) : float_to_bf16_bits(x0[i]);
                const uint32_t hi = dt == DT_F16 ? float_to_half_bits(x1[i]) : float_to_bf16_bits(x1[i]);
                // (the cache's own type: the bits as they came; the other 16-bit type: converted)
                reinterpret_cast<uint32_t*>(dst)[p] = dt == QDT ? reinterpret_cast<const uint32_t*>(src)[p] : (lo | (hi << 16));
            }
        }
        return;
    }
    mn = wave_min(mn);
    mx = wave_max(mx);
    const float levels = dt == DT_U8 ? 255.0f : 15.0f;
    float scale = (mx - mn) / levels;
    if (scale == 0.0f) scale = 0.0001f;
    const float zp = -mn / scale;
    const float inv = 1.0f / scale;
    if (lane == 0) *reinterpret_cast<float2*>(dst) = make_float2(scale, zp);
#pragma unroll
    for (int i = 0; i < PPL; ++i) {
        const int p = lane + 64 * i;
        if (2 * p < D) {
            const float c0 = fminf(fmaxf(rintf(__fmaf_rn(x0[i], inv, zp)), 0.0f), levels);
            const float c1 = fminf(fmaxf(rintf(__fmaf_rn(x1[i], inv, zp)), 0.0f), levels);
            if (dt == DT_U8) reinterpret_cast<uint16_t*>(dst + 8)[p] = (uint16_t)((uint32_t)(int)c0 | ((uint32_t)(int)c1 << 8));
            else dst[8 + p] = (uint8_t)(((uint32_t)(int)c0 << 4) | (uint32_t)(int)c1);
        }
    }
}

template <int QDT>
hipError_t launch_typed(hipStream_t s, const StepDev& st, const GenericShape& sh, const void* query, const void* kc,
                        const void* vc, const int32_t* bi, const AttnWorkspace& ws, void* out, float* scores,
                        int32_t max_kv_len, hipEvent_t ev0, hipEvent_t ev1) {
    const GenericPlan plan = generic_plan(sh, st.T > st.B);
    const int gc = plan.rows, hs = plan.heads;
    const long waves = (long)st.n_gtiles * sh.Hkv * ceil_div(sh.Hq / sh.Hkv, hs) * ws.nsplit;
    if (waves == 0) return hipSuccess;
    auto q = reinterpret_cast<const uint16_t*>(query);
    auto k = reinterpret_cast<const uint8_t*>(kc);
    auto v = reinterpret_cast<const uint8_t*>(vc);
    const dim3 grid((unsigned)((waves + 3) / 4)), block(256);
    const size_t lds = (size_t)4 * gc * sh.Dk * sizeof(float);
    if (ev0) (void)hipEventRecord(ev0, s);
    switch (gc) {
        case 1: hipLaunchKernelGGL((pa_generic_kernel<QDT, 1>), grid, block, lds, s, st, sh, q, k, v, bi, ws, scores ? 1 : 0, hs); break;
        case 2: hipLaunchKernelGGL((pa_generic_kernel<QDT, 2>), grid, block, lds, s, st, sh, q, k, v, bi, ws, scores ? 1 : 0, hs); break;
        case 4: hipLaunchKernelGGL((pa_generic_kernel<QDT, 4>), grid, block, lds, s, st, sh, q, k, v, bi, ws, scores ? 1 : 0, hs); break;
        default: hipLaunchKernelGGL((pa_generic_kernel<QDT, 8>), grid, block, lds, s, st, sh, q, k, v, bi, ws, scores ? 1 : 0, hs); break;
    }
    if (ev1) (void)hipEventRecord(ev1, s);
    const long rows = (long)st.T * sh.Hq;
    hipLaunchKernelGGL((pa_merge_kernel<QDT>), dim3((unsigned)((rows + 3) / 4)), dim3(256), 0, s, st, sh, ws,
                       reinterpret_cast<uint16_t*>(out));
    if (scores) {
        dim3 grid((unsigned)min(ceil_div(max_kv_len, 256), 1024), (unsigned)st.B);
        hipLaunchKernelGGL(pa_scores_single_kernel, grid, dim3(256), 0, s, st, sh, ws, scores);
        if (st.T > st.B)
            hipLaunchKernelGGL((pa_scores_window_kernel<QDT>), grid, dim3(256), 0, s, st, sh, ws, q, k, bi, scores, 0);
    }
    return hipGetLastError();
}

bool generic_shape_ok(const GenericShape& sh) {
    auto dt_ok = [](int dt) { return dt == DT_F16 || dt == DT_BF16 || dt == DT_U8 || dt == DT_U4; };
    return sh.Dk > 0 && sh.Dv > 0 && sh.Dk % 8 == 0 && sh.Dv % 8 == 0 && sh.Dk <= MAX_D && sh.Dv <= MAX_D && dt_ok(sh.kdt) &&
           dt_ok(sh.vdt);
}

}  // namespace

hipError_t launch_attention_generic(hipStream_t s, const StepDev& st, const GenericShape& sh, int q_dtype,
                                    const void* query, const void* key_cache, const void* value_cache,
                                    const int32_t* block_indices, const AttnWorkspace& ws, void* out, float* scores,
                                    int32_t max_kv_len, hipEvent_t ev0, hipEvent_t ev1) {
    if (!generic_shape_ok(sh)) return hipErrorInvalidValue;
    if (q_dtype == DT_F16)
        return launch_typed<DT_F16>(s, st, sh, query, key_cache, value_cache, block_indices, ws, out, scores, max_kv_len, ev0, ev1);
    if (q_dtype == DT_BF16)
        return launch_typed<DT_BF16>(s, st, sh, query, key_cache, value_cache, block_indices, ws, out, scores, max_kv_len, ev0, ev1);
    return hipErrorInvalidValue;
}

// ---- block diversity for every shape (what pa_rkv_diversity.hip does on the matrix cores for its shapes) ----------
// out[block][c] = -(1 / Hkv) * sum over kv heads and over the block's rows r of cos(k_r, k_c), with the diagonal set
// to zero and entries below their row's mean (over the whole area) dropped.  Three passes over the area's key rows,
// every sum in a fixed order:
//   1. per token: 1 / |k| -> `stats[..].x` (and k^ . k^ -> .w); per chunk of 256 tokens the column sums of k^ -> `colsum`;
//   2. per token: the row's mean -> `mean`, from k^_r . (sum over the area of k^) - k^_r . k^_r;
//   3. per (block, 64 columns): the similarities, 16 rows of k^ at a time through LDS.
namespace {
constexpr int GDIV_CHUNK = 256;
constexpr float GDIV_EPS = 1e-12f;

// The lane's eight channels (8 lane ..) of token j of the area, as floats; lanes beyond the row get zeros.
__device__ __forceinline__ void gdiv_load(const RkvDivArgs& a, const RkvDivSeq& q, const int32_t* table, int h, int j,
                                          int D, int bs, int dt, int lane, float (&x)[8]) {
    const int pos = q.first_block * bs + j;
    RowReader rr(a.key_cache, table[pos / bs], h, pos % bs, a.Hkv, bs, D, dt);
    if (8 * lane < D) {
        rr.load8(8 * lane, x);
    } else {
#pragma unroll
        for (int e = 0; e < 8; ++e) x[e] = 0.0f;
    }
}

__global__ __launch_bounds__(256) void gdiv_norm_colsum_kernel(RkvDivArgs a, int D, int bs, int dt) {
    __shared__ float red[4][MAX_D];
    const RkvDivSeq q = a.seqs[blockIdx.z];
    const int h = blockIdx.y, base = blockIdx.x * GDIV_CHUNK;
    if (base >= q.ev) return;
    const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
    const int32_t* table = a.block_indices + q.table_off;
    float acc[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[e] = 0.0f;
    for (int j = base + wv; j < min(base + GDIV_CHUNK, q.ev); j += 4) {  // (wave-uniform bounds)
        float x[8];
        gdiv_load(a, q, table, h, j, D, bs, dt, lane, x);
        float sq = 0.0f;
#pragma unroll
        for (int e = 0; e < 8; ++e) sq = fmaf(x[e], x[e], sq);
        sq = wave_sum(sq);
        const float inv = 1.0f / sqrtf(sq + GDIV_EPS);
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[e] = fmaf(x[e], inv, acc[e]);
        if (lane == 0) a.stats[(long)h * a.total_tok + q.tok_off + j] = make_float4(inv, 0.0f, 0.0f, sq * inv * inv);
    }
    if (8 * lane < D) {
#pragma unroll
        for (int e = 0; e < 8; ++e) red[wv][8 * lane + e] = acc[e];
    }
    __syncthreads();
    for (int d = threadIdx.x; d < D; d += 256)
        a.colsum[(((long)blockIdx.z * a.Hkv + h) * (a.chunks_max + 1) + 1 + blockIdx.x) * D + d] =
            ((red[0][d] + red[1][d]) + red[2][d]) + red[3][d];
}

__global__ __launch_bounds__(256) void gdiv_total_kernel(RkvDivArgs a, int D) {
    const RkvDivSeq q = a.seqs[blockIdx.y];
    const int chunks = (q.ev + GDIV_CHUNK - 1) / GDIV_CHUNK;
    float* cs = a.colsum + ((long)blockIdx.y * a.Hkv + blockIdx.x) * (a.chunks_max + 1) * D;
    for (int d = threadIdx.x; d < D; d += 256) {
        float s = 0.0f;
        for (int c = 0; c < chunks; ++c) s += cs[(long)(1 + c) * D + d];
        cs[d] = s;
    }
}

__global__ __launch_bounds__(256) void gdiv_mean_kernel(RkvDivArgs a, int D, int bs, int dt) {
    const RkvDivSeq q = a.seqs[blockIdx.z];
    const int h = blockIdx.y;
    const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
    const int j = blockIdx.x * 4 + wv;
    if (j >= q.ev) return;  // (wave-uniform)
    const int32_t* table = a.block_indices + q.table_off;
    const float* tot = a.colsum + ((long)blockIdx.z * a.Hkv + h) * (a.chunks_max + 1) * D;
    float x[8];
    gdiv_load(a, q, table, h, j, D, bs, dt, lane, x);
    float d = 0.0f;
    if (8 * lane < D) {
#pragma unroll
        for (int e = 0; e < 8; ++e) d = fmaf(x[e], tot[8 * lane + e], d);
    }
    d = wave_sum(d);
    const float4 st = a.stats[(long)h * a.total_tok + q.tok_off + j];
    if (lane == 0) a.mean[(long)h * a.total_tok + q.tok_off + j] = (d * st.x - st.w) / (float)q.ev;
}

// A workgroup = one block of rows x 64 columns: thread (column c of the 64, quarter qd) holds its column's row of one
// kv head in registers, D elements at most 128 at a time, and meets rows 4 * i + qd of every 16-row slice of the block
// in LDS.
__global__ __launch_bounds__(256) void gdiv_pair_kernel(RkvDivArgs a, int D, int bs, int dt) {
    __shared__ __align__(16) float rows[16][128 + 4];
    __shared__ float rmean[16], part[4][64];
    const RkvDivSeq q = a.seqs[blockIdx.z];
    const int rb = blockIdx.y;
    if (rb * bs >= q.ev || (int)blockIdx.x * 64 >= q.ev) return;
    const int cl = threadIdx.x & 63, qd = threadIdx.x >> 6;
    const int c = blockIdx.x * 64 + cl;
    const bool col_ok = c < q.ev;
    const int cj = min(c, q.ev - 1);
    const int32_t* table = a.block_indices + q.table_off;
    float total = 0.0f;
    for (int h = 0; h < a.Hkv; ++h) {
        const long sbase = (long)h * a.total_tok + q.tok_off;
        const float c_inv = a.stats[sbase + cj].x;
        const int cpos = q.first_block * bs + cj;
        RowReader cr(a.key_cache, table[cpos / bs], h, cpos % bs, a.Hkv, bs, D, dt);
        const int rend = (rb + 1) * bs;
        for (int r0 = rb * bs; r0 < rend; r0 += 16) {  // (a last slice may hold fewer than 16 rows: the others are zeros that count for nothing)
            float dot[4] = {0.0f, 0.0f, 0.0f, 0.0f};
            for (int d0 = 0; d0 < D; d0 += 128) {
                const int dn = min(128, D - d0);
                __syncthreads();  // the slice staged before is done with
                // stage rows r0 .. r0 + 15, channels d0 .. d0 + dn - 1, as k^ (thread t: row t / 16, eight channels)
                {
                    const int rr_ = threadIdx.x >> 4, ch = (threadIdx.x & 15) * 8;
                    if (ch < dn) {
                        const int rj = min(r0 + rr_, rend - 1);
                        const int rpos = q.first_block * bs + rj;
                        RowReader rr(a.key_cache, table[rpos / bs], h, rpos % bs, a.Hkv, bs, D, dt);
                        float x[8];
                        rr.load8(d0 + ch, x);
                        const float inv = r0 + rr_ < rend ? a.stats[sbase + rj].x : 0.0f;
#pragma unroll
                        for (int e = 0; e < 8; ++e) rows[rr_][ch + e] = x[e] * inv;
                    }
                    if (d0 == 0 && threadIdx.x < 16)
                        rmean[threadIdx.x] = r0 + (int)threadIdx.x < rend ? a.mean[sbase + r0 + threadIdx.x] : INFINITY;
                }
                __syncthreads();
                for (int d = 0; d < dn; d += 8) {
                    float y[8];
                    cr.load8(d0 + d, y);
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        const float4 ra = *reinterpret_cast<const float4*>(&rows[4 * i + qd][d]);
                        const float4 rb4 = *reinterpret_cast<const float4*>(&rows[4 * i + qd][d + 4]);
                        dot[i] = fmaf(y[0], ra.x, dot[i]); dot[i] = fmaf(y[1], ra.y, dot[i]);
                        dot[i] = fmaf(y[2], ra.z, dot[i]); dot[i] = fmaf(y[3], ra.w, dot[i]);
                        dot[i] = fmaf(y[4], rb4.x, dot[i]); dot[i] = fmaf(y[5], rb4.y, dot[i]);
                        dot[i] = fmaf(y[6], rb4.z, dot[i]); dot[i] = fmaf(y[7], rb4.w, dot[i]);
                    }
                }
            }
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int r = r0 + 4 * i + qd;
                const float v = r == c ? 0.0f : dot[i] * c_inv;
                total += v < rmean[4 * i + qd] ? 0.0f : v;
            }
        }
    }
    __syncthreads();
    part[qd][cl] = total;
    __syncthreads();
    if (qd == 0 && col_ok)
        a.out[q.out_off + (long)rb * q.ev + c] = -((((part[0][cl] + part[1][cl]) + part[2][cl]) + part[3][cl]) / (float)a.Hkv);
}
}  // namespace

hipError_t launch_rkv_diversity_generic(hipStream_t s, const RkvDivArgs& a, int kv_dtype, int D, int bs, int nseq, int ev_max) {
    if (nseq == 0 || ev_max == 0) return hipSuccess;
    if (D <= 0 || D > MAX_D || D % 8 || bs <= 0 || ev_max % bs) return hipErrorInvalidValue;
    const int chunks = (ev_max + GDIV_CHUNK - 1) / GDIV_CHUNK;
    if (chunks > a.chunks_max) return hipErrorInvalidValue;
    hipLaunchKernelGGL(gdiv_norm_colsum_kernel, dim3((unsigned)chunks, (unsigned)a.Hkv, (unsigned)nseq), dim3(256), 0, s, a, D, bs, kv_dtype);
    hipLaunchKernelGGL(gdiv_total_kernel, dim3((unsigned)a.Hkv, (unsigned)nseq), dim3(256), 0, s, a, D);
    hipLaunchKernelGGL(gdiv_mean_kernel, dim3((unsigned)((ev_max + 3) / 4), (unsigned)a.Hkv, (unsigned)nseq), dim3(256), 0, s, a, D, bs, kv_dtype);
    hipLaunchKernelGGL(gdiv_pair_kernel, dim3((unsigned)((ev_max + 63) / 64), (unsigned)(ev_max / bs), (unsigned)nseq), dim3(256), 0, s, a, D, bs, kv_dtype);
    return hipGetLastError();
}

hipError_t launch_kv_append_generic(hipStream_t s, const StepDev& st, const GenericShape& sh, int q_dtype, const void* key,
                                    const void* value, void* key_cache, void* value_cache, const int32_t* block_indices) {
    if (!generic_shape_ok(sh)) return hipErrorInvalidValue;
    const long rows = (long)st.T * sh.Hkv * 2;
    if (rows == 0) return hipSuccess;
    auto k = reinterpret_cast<const uint16_t*>(key);
    auto v = reinterpret_cast<const uint16_t*>(value);
    auto kc = reinterpret_cast<uint8_t*>(key_cache);
    auto vc = reinterpret_cast<uint8_t*>(value_cache);
    const dim3 grid((unsigned)((rows + 3) / 4));
    if (q_dtype == DT_F16) hipLaunchKernelGGL((kv_append_generic_kernel<DT_F16>), grid, dim3(256), 0, s, st, sh, k, v, kc, vc, block_indices);
    else if (q_dtype == DT_BF16) hipLaunchKernelGGL((kv_append_generic_kernel<DT_BF16>), grid, dim3(256), 0, s, st, sh, k, v, kc, vc, block_indices);
    else return hipErrorInvalidValue;
    return hipGetLastError();
}

}  // namespace pa
