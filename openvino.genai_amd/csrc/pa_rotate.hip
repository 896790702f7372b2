// Cache rotation: after blocks have been evicted from the middle of a sequence, the K rows of the blocks behind
// them are re-rotated in place so that their rotary position matches their new place in the sequence.
//
// Element pairs (j, j + D/2) of a (rotated block, kv head, token) row are rotated as in rotate_half RoPE with the
// table row the block's (or token's) delta selects:
//     x' = cos * x - sin * y,   y' = cos * y + sin * x        (the table's sines carry the minus sign)
// products and sums rounded separately in binary32 (no contraction) so that the bytes are reproducible on any
// IEEE host.  16-bit rows are rounded back to their type; u8 rows are dequantised, rotated and quantised again
// with the row recipe (row min / max, scale, zero-point, codes).  HBM-bound byte work: each row is read and
// written once, plus one table row per row (shared by the block's rows, so served from cache).
//
// Head sizes 64 and 128: eight lanes own a row, D / 16 pairs each (8- or 16-byte accesses at D = 128), eight rows
// per wave, rows in the order they lie in the cache (block, kv head, token), so a workgroup's 32 rows are one run of
// bytes; row minimum and maximum by three cross-lane steps.  (Sixteen lanes per row: 25 % slower over u8 rows, whose
// per-row arithmetic -- three divisions, the reductions -- every lane repeats; four lanes per row: the same within
// 2 %.)  Other even head sizes up to 128: a wave per row, one pair per lane.
#include "pa_device.h"

namespace pa {
namespace {

// A wave per row, PPL pairs per lane: head sizes up to 128 * PPL (lanes beyond half a row idle).
template <int KVDT, int PPL>
__global__ __launch_bounds__(256) void pa_rotate_kernel(uint8_t* __restrict__ key_cache, Shape sh,
                                                        const int32_t* __restrict__ rotated_block_indices,
                                                        const int32_t* __restrict__ deltas, int32_t deltas_per_block,
                                                        int32_t n_rotated, const float* __restrict__ trig_lut) {
#pragma clang fp contract(off)
    const int lane = threadIdx.x & 63;
    const long row = (long)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= (long)n_rotated * sh.bs * sh.Hkv) return;
    const int h = (int)(row % sh.Hkv);
    const int t = (int)((row / sh.Hkv) % sh.bs);
    const int i = (int)(row / ((long)sh.Hkv * sh.bs));
    const int D = sh.D, half = D / 2;
    const long phys = rotated_block_indices[i];
    const int delta = deltas[(long)i * deltas_per_block + (deltas_per_block == 1 ? 0 : t)];
    const float* cs = trig_lut + (long)delta * D;
    const float* sn = cs + half;
    uint8_t* dst = key_cache + ((phys * sh.Hkv + h) * sh.bs + t) * (long)row_bytes(D, KVDT);
    const bool on = lane * PPL < half;

    float x[PPL], y[PPL];
    if (KVDT == DT_U8) {
        const float2 hd = *reinterpret_cast<const float2*>(dst);
#pragma unroll
        for (int e = 0; e < PPL; ++e) {
            const int j = lane * PPL + e;
            x[e] = on ? ((float)dst[8 + j] - hd.y) * hd.x : 0.0f;
            y[e] = on ? ((float)dst[8 + half + j] - hd.y) * hd.x : 0.0f;
        }
    } else {
        const uint16_t* r16 = reinterpret_cast<const uint16_t*>(dst);
#pragma unroll
        for (int e = 0; e < PPL; ++e) {
            const int j = lane * PPL + e;
            x[e] = on ? load16<KVDT>(r16[j]) : 0.0f;
            y[e] = on ? load16<KVDT>(r16[half + j]) : 0.0f;
        }
    }
    float nx[PPL], ny[PPL];
#pragma unroll
    for (int e = 0; e < PPL; ++e) {
        const int j = lane * PPL + e;
        const float c = on ? cs[j] : 1.0f, s = on ? sn[j] : 0.0f;
        // plain operators: the contract(off) pragma above covers them (it does not reach into inlined intrinsics)
        const float xc = x[e] * c, ys = y[e] * s, yc = y[e] * c, xs = x[e] * s;
        nx[e] = xc - ys;
        ny[e] = yc + xs;
    }
    if (KVDT == DT_U8) {
        float mn = INFINITY, mx = -INFINITY;
        if (on) {
#pragma unroll
            for (int e = 0; e < PPL; ++e) {
                mn = fminf(mn, fminf(nx[e], ny[e]));
                mx = fmaxf(mx, fmaxf(nx[e], ny[e]));
            }
        }
        mn = wave_min(mn);
        mx = wave_max(mx);
        float scale = (mx - mn) / 255.0f;
        if (scale == 0.0f) scale = 0.0001f;
        const float zp = -mn / scale;
        const float inv = 1.0f / scale;
        if (lane == 0) *reinterpret_cast<float2*>(dst) = make_float2(scale, zp);
        if (on) {
#pragma unroll
            for (int e = 0; e < PPL; ++e) {
                const int j = lane * PPL + e;
                float a = rintf(__fmaf_rn(nx[e], inv, zp)), b = rintf(__fmaf_rn(ny[e], inv, zp));
                a = fminf(fmaxf(a, 0.0f), 255.0f);
                b = fminf(fmaxf(b, 0.0f), 255.0f);
                dst[8 + j] = (uint8_t)(int)a;
                dst[8 + half + j] = (uint8_t)(int)b;
            }
        }
    } else if (on) {
        uint16_t* r16 = reinterpret_cast<uint16_t*>(dst);
#pragma unroll
        for (int e = 0; e < PPL; ++e) {
            const int j = lane * PPL + e;
            r16[j] = store16<KVDT>(nx[e]);
            r16[half + j] = store16<KVDT>(ny[e]);
        }
    }
}

// LPR lanes own a row, E = D / (2 LPR) pairs each: the lane's x elements are E consecutive ones of the row's first
// half, its y elements the E at the same place of the second half.
template <int KVDT, int E, int LPR>
__global__ __launch_bounds__(256) void pa_rotate_rows_kernel(uint8_t* __restrict__ key_cache, Shape sh,
                                                             const int32_t* __restrict__ rotated_block_indices,
                                                             const int32_t* __restrict__ deltas, int32_t deltas_per_block,
                                                             int32_t n_rotated, const float* __restrict__ trig_lut) {
#pragma clang fp contract(off)
    static_assert(E % 4 == 0 && LPR == 8, "whole words of codes per lane; the row reductions below take three steps");
    constexpr int HALF = LPR * E, D = 2 * HALF;
    constexpr int ROWB = KVDT == DT_U8 ? D + 8 : D * 2;
    typedef uint32_t u8w __attribute__((ext_vector_type(E / 4)));   // E codes
    typedef uint32_t u16w __attribute__((ext_vector_type(E / 2)));  // E 16-bit elements
    typedef float fE __attribute__((ext_vector_type(E)));
    const int l = threadIdx.x % LPR;
    const long n_rows = (long)n_rotated * sh.Hkv * sh.bs;
    long row = (long)blockIdx.x * (256 / LPR) + threadIdx.x / LPR;
    const bool live = row < n_rows;
    row = min(row, n_rows - 1);  // (surplus groups repeat the last row and store nothing: every lane takes the cross-lane steps)
    const int t = (int)(row % sh.bs);
    const int i = (int)(row / ((long)sh.Hkv * sh.bs));
    const long phys = rotated_block_indices[i];
    const int delta = deltas[(long)i * deltas_per_block + (deltas_per_block == 1 ? 0 : t)];
    const fE cs = *reinterpret_cast<const fE*>(trig_lut + (long)delta * D + l * E);
    const fE sn = *reinterpret_cast<const fE*>(trig_lut + (long)delta * D + HALF + l * E);
    // row = (i * Hkv + h) * bs + t: the row's place within the listed blocks is its place within block `phys`
    uint8_t* dst = key_cache + (phys * sh.Hkv * sh.bs + row % ((long)sh.Hkv * sh.bs)) * ROWB;

    float x[E], y[E];
    if (KVDT == DT_U8) {
        const float2 hd = *reinterpret_cast<const float2*>(dst);
        const u8w wx = *reinterpret_cast<const u8w*>(dst + 8 + E * l);
        const u8w wy = *reinterpret_cast<const u8w*>(dst + 8 + HALF + E * l);
#pragma unroll
        for (int e = 0; e < E; ++e) {
            x[e] = ((float)((wx[e / 4] >> (8 * (e % 4))) & 0xffu) - hd.y) * hd.x;
            y[e] = ((float)((wy[e / 4] >> (8 * (e % 4))) & 0xffu) - hd.y) * hd.x;
        }
    } else {
        const u16w wx = *reinterpret_cast<const u16w*>(dst + 2 * E * l);
        const u16w wy = *reinterpret_cast<const u16w*>(dst + 2 * HALF + 2 * E * l);
#pragma unroll
        for (int e = 0; e < E; ++e) {
            x[e] = load16<KVDT>((uint16_t)(wx[e / 2] >> (16 * (e % 2))));
            y[e] = load16<KVDT>((uint16_t)(wy[e / 2] >> (16 * (e % 2))));
        }
    }
    float nx[E], ny[E];
#pragma unroll
    for (int e = 0; e < E; ++e) {
        const float c = cs[e], s = sn[e];
        // plain operators: the contract(off) pragma above covers them (it does not reach into inlined intrinsics)
        const float xc = x[e] * c, ys = y[e] * s, yc = y[e] * c, xs = x[e] * s;
        nx[e] = xc - ys;
        ny[e] = yc + xs;
    }
    if (KVDT == DT_U8) {
        float mn = INFINITY, mx = -INFINITY;
#pragma unroll
        for (int e = 0; e < E; ++e) {
            mn = fminf(mn, fminf(nx[e], ny[e]));
            mx = fmaxf(mx, fmaxf(nx[e], ny[e]));
        }
        mn = row8_min(mn);
        mx = row8_max(mx);
        float scale = (mx - mn) / 255.0f;
        if (scale == 0.0f) scale = 0.0001f;
        const float zp = -mn / scale;
        const float inv = 1.0f / scale;
        u8w wx, wy;
#pragma unroll
        for (int w = 0; w < E / 4; ++w) wx[w] = wy[w] = 0u;
#pragma unroll
        for (int e = 0; e < E; ++e) {
            float a = rintf(__fmaf_rn(nx[e], inv, zp)), b = rintf(__fmaf_rn(ny[e], inv, zp));
            a = fminf(fmaxf(a, 0.0f), 255.0f);
            b = fminf(fmaxf(b, 0.0f), 255.0f);
            wx[e / 4] |= (uint32_t)(int)a << (8 * (e % 4));
            wy[e / 4] |= (uint32_t)(int)b << (8 * (e % 4));
        }
        if (!live) return;
        if (l == 0) *reinterpret_cast<float2*>(dst) = make_float2(scale, zp);
        *reinterpret_cast<u8w*>(dst + 8 + E * l) = wx;
        *reinterpret_cast<u8w*>(dst + 8 + HALF + E * l) = wy;
    } else {
        if (!live) return;
        u16w wx, wy;
#pragma unroll
        for (int e = 0; e < E / 2; ++e) {
            wx[e] = (uint32_t)store16<KVDT>(nx[2 * e]) | ((uint32_t)store16<KVDT>(nx[2 * e + 1]) << 16);
            wy[e] = (uint32_t)store16<KVDT>(ny[2 * e]) | ((uint32_t)store16<KVDT>(ny[2 * e + 1]) << 16);
        }
        *reinterpret_cast<u16w*>(dst + 2 * E * l) = wx;
        *reinterpret_cast<u16w*>(dst + 2 * HALF + 2 * E * l) = wy;
    }
}

template <int KVDT>
hipError_t launch_ppl(hipStream_t s, uint8_t* kc, const Shape& sh, const int32_t* idx, const int32_t* deltas,
                      int32_t deltas_per_block, int32_t n, const float* lut) {
    const long rows = (long)n * sh.bs * sh.Hkv;
    const dim3 grid((unsigned)((rows + 3) / 4)), block(256);
    if (sh.D > 512 || sh.D % 8) return hipErrorInvalidValue;  // (half a row is a whole number of pairs per lane below)
    if (sh.D == 256 || sh.D == 128 || sh.D == 64) {
        if (sh.D == 256)
            hipLaunchKernelGGL((pa_rotate_rows_kernel<KVDT, 16, 8>), dim3((unsigned)((rows + 31) / 32)), block, 0, s, kc, sh, idx, deltas, deltas_per_block, n, lut);
        else if (sh.D == 128)
            hipLaunchKernelGGL((pa_rotate_rows_kernel<KVDT, 8, 8>), dim3((unsigned)((rows + 31) / 32)), block, 0, s, kc, sh, idx, deltas, deltas_per_block, n, lut);
        else
            hipLaunchKernelGGL((pa_rotate_rows_kernel<KVDT, 4, 8>), dim3((unsigned)((rows + 31) / 32)), block, 0, s, kc, sh, idx, deltas, deltas_per_block, n, lut);
        return hipGetLastError();
    }
    if (sh.D <= 128) hipLaunchKernelGGL((pa_rotate_kernel<KVDT, 1>), grid, block, 0, s, kc, sh, idx, deltas, deltas_per_block, n, lut);
    else if (sh.D <= 256) hipLaunchKernelGGL((pa_rotate_kernel<KVDT, 2>), grid, block, 0, s, kc, sh, idx, deltas, deltas_per_block, n, lut);
    else hipLaunchKernelGGL((pa_rotate_kernel<KVDT, 4>), grid, block, 0, s, kc, sh, idx, deltas, deltas_per_block, n, lut);
    return hipGetLastError();
}

}  // namespace

hipError_t launch_rotate(hipStream_t s, void* key_cache, int kv_dtype, const Shape& sh,
                         const int32_t* rotated_block_indices, const int32_t* deltas, int32_t deltas_per_block,
                         int32_t n_rotated, const float* trig_lut) {
    if (n_rotated == 0) return hipSuccess;
    auto kc = static_cast<uint8_t*>(key_cache);
    if (kv_dtype == DT_U8) return launch_ppl<DT_U8>(s, kc, sh, rotated_block_indices, deltas, deltas_per_block, n_rotated, trig_lut);
    if (kv_dtype == DT_F16) return launch_ppl<DT_F16>(s, kc, sh, rotated_block_indices, deltas, deltas_per_block, n_rotated, trig_lut);
    return launch_ppl<DT_BF16>(s, kc, sh, rotated_block_indices, deltas, deltas_per_block, n_rotated, trig_lut);
}

}  // namespace pa
