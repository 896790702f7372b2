// KV append: writes the new tokens' K and V rows into the block-tabled caches.
//
// Sixteen lanes own one (token, kv head, K|V) row of D elements, so the row's min/max is a reduction over 16 lanes
// and a wave writes four rows.  HBM-bound byte work: each input element is read once and each cache byte written
// once.
//
// u8 rows are `f32 scale | f32 zero-point | D codes` with
//   scale = (max - min) / 255  (a zero range takes 1e-4),  zp = -min / scale,
//   code  = clamp(rne(fma(x, 1/scale, zp)), 0, 255),
// every operation in IEEE binary32 so that the bytes are reproducible on any IEEE host.
#include "pa_device.h"

namespace pa {
namespace {

constexpr int TOKENS_KERNEL_MIN_T = 8192;  // steps of this many tokens take the kernel that walks a token's rows

// One row's 16 lanes: `w` holds the lane's E elements as loaded, `dst` is the row in the cache.
template <int QDT, int KVDT, int E>
__device__ __forceinline__ void append_row(uint32_t (&w)[E / 2], uint8_t* dst, int l16) {
#pragma clang fp contract(off)
    if constexpr (KVDT == DT_U8) {
        float x[E];
#pragma unroll
        for (int e = 0; e < E; ++e) x[e] = load16<QDT>((uint16_t)(w[e / 2] >> (16 * (e & 1))));
        float mn = x[0], mx = x[0];
#pragma unroll
        for (int e = 1; e < E; ++e) { mn = fminf(mn, x[e]); mx = fmaxf(mx, x[e]); }
        mn = row16_min(mn);
        mx = row16_max(mx);
        float scale = (mx - mn) / 255.0f;
        if (scale == 0.0f) scale = 0.0001f;
        const float zp = -mn / scale;
        const float inv = 1.0f / scale;
        uint32_t codes[(E + 3) / 4];
#pragma unroll
        for (int i = 0; i < (E + 3) / 4; ++i) codes[i] = 0;
#pragma unroll
        for (int e = 0; e < E; ++e) {
            float v = rintf(__fmaf_rn(x[e], inv, zp));
            v = fminf(fmaxf(v, 0.0f), 255.0f);
            codes[e / 4] |= (uint32_t)(int)v << (8 * (e & 3));
        }
        if (l16 == 0) *reinterpret_cast<float2*>(dst) = make_float2(scale, zp);
        uint8_t* c = dst + 8 + l16 * E;  // rows are multiples of 8 bytes
        if constexpr (E == 4) *reinterpret_cast<uint32_t*>(c) = codes[0];
        else if constexpr (E == 6) {  // (a lane's six bytes start on a 2-byte boundary)
            reinterpret_cast<uint16_t*>(c)[0] = (uint16_t)codes[0];
            reinterpret_cast<uint16_t*>(c)[1] = (uint16_t)(codes[0] >> 16);
            reinterpret_cast<uint16_t*>(c)[2] = (uint16_t)codes[1];
        } else
#pragma unroll
            for (int i = 0; i < E / 8; ++i) *reinterpret_cast<uint2*>(c + 8 * i) = make_uint2(codes[2 * i], codes[2 * i + 1]);
    } else {
        if constexpr (QDT != KVDT) {
#pragma unroll
            for (int i = 0; i < E / 2; ++i)
                w[i] = (uint32_t)store16<KVDT>(load16<QDT>((uint16_t)(w[i] & 0xffff))) |
                       ((uint32_t)store16<KVDT>(load16<QDT>((uint16_t)(w[i] >> 16))) << 16);
        }
        uint8_t* c = dst + l16 * E * 2;
        if constexpr (E == 4) *reinterpret_cast<uint2*>(c) = make_uint2(w[0], w[1]);
        else if constexpr (E == 6) {  // (twelve bytes on a 4-byte boundary)
#pragma unroll
            for (int i = 0; i < 3; ++i) reinterpret_cast<uint32_t*>(c)[i] = w[i];
        } else
#pragma unroll
            for (int i = 0; i < E / 8; ++i) *reinterpret_cast<uint4*>(c + 16 * i) = make_uint4(w[4 * i], w[4 * i + 1], w[4 * i + 2], w[4 * i + 3]);
    }
}

template <int E>
__device__ __forceinline__ void load_row(uint32_t (&w)[E / 2], const uint16_t* src) {
    if constexpr (E == 4) {
        const uint2 v = *reinterpret_cast<const uint2*>(src);
        w[0] = v.x; w[1] = v.y;
    } else if constexpr (E == 6) {
#pragma unroll
        for (int i = 0; i < 3; ++i) w[i] = reinterpret_cast<const uint32_t*>(src)[i];
    } else {
#pragma unroll
        for (int i = 0; i < E / 8; ++i) {
            const uint4 v = *reinterpret_cast<const uint4*>(src + 8 * i);
            w[4 * i] = v.x; w[4 * i + 1] = v.y; w[4 * i + 2] = v.z; w[4 * i + 3] = v.w;
        }
    }
}

// A row per 16 lanes, each lane D / 16 consecutive elements (16-byte loads at D = 128 and 256, 4-byte ones at 96),
// four rows per wave.  A wave
// takes four consecutive tokens of one kv head, so that what it writes is one run of cache bytes wherever the
// tokens share a block.  Minimum and maximum of a row are reduced over its 16 lanes with four
// cross-lane (DPP) steps; the arithmetic per element is that of quantize_row_u8, so the bytes are the same.
template <int QDT, int KVDT, int E>
__global__ __launch_bounds__(256) void kv_append_kernel(StepDev st, Shape sh, const uint16_t* __restrict__ key,
                                                        const uint16_t* __restrict__ value,
                                                        uint8_t* __restrict__ key_cache,
                                                        uint8_t* __restrict__ value_cache,
                                                        const int32_t* __restrict__ block_indices) {
#pragma clang fp contract(off)
    static_assert(E == 4 || E == 6 || E == 8 || E == 16, "D = 64, 96, 128 or 256");
    constexpr int D = 16 * E;
    const int l16 = threadIdx.x & 15;
    const long per_tensor = (long)st.T * sh.Hkv;
    long row = ((long)blockIdx.x * 256 + threadIdx.x) >> 4;  // (K | V, kv head, token)
    // (rows beyond the end repeat the last one: no divergence around the cross-lane steps, and the same bytes twice)
    row = min(row, 2 * per_tensor - 1);
    const int which = row >= per_tensor;
    const long rem = row - which * per_tensor;
    const int h = (int)(rem / st.T), t = (int)(rem % st.T);
    const int b = st.token_seq[t];
    const int slot = st.past_lens[b] + (t - st.subsequence_begins[b]);
    const long phys = block_indices[st.block_indices_begins[b] + slot / sh.bs];
    constexpr int RB = KVDT == DT_U8 ? D + 8 : 2 * D;
    const uint16_t* src = (which ? value : key) + ((long)t * sh.Hkv + h) * D + l16 * E;
    uint8_t* dst = (which ? value_cache : key_cache) + ((phys * sh.Hkv + h) * sh.bs + slot % sh.bs) * (long)RB;

    uint32_t w[E / 2];
    load_row<E>(w, src);
    append_row<QDT, KVDT, E>(w, dst, l16);
}

// Steps of many tokens (a prompt's chunk): sixteen lanes own one TOKEN and walk its 2 * Hkv rows (K then V, kv heads
// in order), four rows' loads in flight.  The chain of dependent loads that leads to a row's place in the cache
// (token -> sequence -> position -> block id) is walked once per token instead of once per row, and a lane has four
// times the bytes in flight: with a row per 16 lanes that chain, not the memory system, set the pace (3.2 TB/s into a
// u8 cache at 131072 tokens x 8 kv heads).
template <int QDT, int KVDT, int E>
__global__ __launch_bounds__(256) void kv_append_tokens_kernel(StepDev st, Shape sh, const uint16_t* __restrict__ key,
                                                               const uint16_t* __restrict__ value,
                                                               uint8_t* __restrict__ key_cache,
                                                               uint8_t* __restrict__ value_cache,
                                                               const int32_t* __restrict__ block_indices) {
    static_assert(E == 4 || E == 6 || E == 8 || E == 16, "D = 64, 96, 128 or 256");
    constexpr int D = 16 * E, U = 4;
    constexpr int RB = KVDT == DT_U8 ? D + 8 : 2 * D;
    const int l16 = threadIdx.x & 15;
    // (tokens beyond the end repeat the last one: no divergence around the cross-lane steps, and the same bytes twice)
    const int t = min((int)blockIdx.x * 16 + (int)(threadIdx.x >> 4), st.T - 1);
    const int b = st.token_seq[t];
    const int slot = st.past_lens[b] + (t - st.subsequence_begins[b]);
    const long phys = block_indices[st.block_indices_begins[b] + slot / sh.bs];
    const long dst_tok = (phys * sh.Hkv * sh.bs + slot % sh.bs) * (long)RB;  // the token's row of kv head 0
    const long head_stride = (long)sh.bs * RB;
    const uint16_t* src_tok = nullptr;
    const int rows = 2 * sh.Hkv;
    for (int j0 = 0; j0 < rows; j0 += U) {
        uint32_t w[U][E / 2];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int j = min(j0 + u, rows - 1);  // (a last group that is not full repeats the last row)
            const int which = j >= sh.Hkv, h = j - which * sh.Hkv;
            src_tok = (which ? value : key) + ((long)t * sh.Hkv + h) * D + l16 * E;
            load_row<E>(w[u], src_tok);
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int j = min(j0 + u, rows - 1);
            const int which = j >= sh.Hkv, h = j - which * sh.Hkv;
            append_row<QDT, KVDT, E>(w[u], (which ? value_cache : key_cache) + dst_tok + h * head_stride, l16);
        }
    }
}

template <int QDT, int KVDT>
hipError_t launch_epl(hipStream_t s, const StepDev& st, const Shape& sh, const void* key, const void* value,
                      void* kc, void* vc, const int32_t* bi) {
    const long rows = (long)st.T * sh.Hkv * 2;
    if (rows == 0) return hipSuccess;
    dim3 grid((unsigned)((rows + 15) / 16)), block(256);
    auto k = reinterpret_cast<const uint16_t*>(key);
    auto v = reinterpret_cast<const uint16_t*>(value);
    auto kcu = reinterpret_cast<uint8_t*>(kc);
    auto vcu = reinterpret_cast<uint8_t*>(vc);
    if (st.T >= TOKENS_KERNEL_MIN_T) {  // enough tokens to fill the chip with a token per 16 lanes
        const dim3 tgrid((unsigned)((st.T + 15) / 16));
        switch (sh.D) {
            case 64: hipLaunchKernelGGL((kv_append_tokens_kernel<QDT, KVDT, 4>), tgrid, block, 0, s, st, sh, k, v, kcu, vcu, bi); break;
            case 96: hipLaunchKernelGGL((kv_append_tokens_kernel<QDT, KVDT, 6>), tgrid, block, 0, s, st, sh, k, v, kcu, vcu, bi); break;
            case 128: hipLaunchKernelGGL((kv_append_tokens_kernel<QDT, KVDT, 8>), tgrid, block, 0, s, st, sh, k, v, kcu, vcu, bi); break;
            case 256: hipLaunchKernelGGL((kv_append_tokens_kernel<QDT, KVDT, 16>), tgrid, block, 0, s, st, sh, k, v, kcu, vcu, bi); break;
            default: return hipErrorInvalidValue;
        }
        return hipGetLastError();
    }
    switch (sh.D) {
        case 64: hipLaunchKernelGGL((kv_append_kernel<QDT, KVDT, 4>), grid, block, 0, s, st, sh, k, v, kcu, vcu, bi); break;
        case 96: hipLaunchKernelGGL((kv_append_kernel<QDT, KVDT, 6>), grid, block, 0, s, st, sh, k, v, kcu, vcu, bi); break;
        case 128: hipLaunchKernelGGL((kv_append_kernel<QDT, KVDT, 8>), grid, block, 0, s, st, sh, k, v, kcu, vcu, bi); break;
        case 256: hipLaunchKernelGGL((kv_append_kernel<QDT, KVDT, 16>), grid, block, 0, s, st, sh, k, v, kcu, vcu, bi); break;
        default: return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

}  // namespace

hipError_t launch_kv_append(hipStream_t s, const StepDev& st, const Shape& sh, int q_dtype, int kv_dtype,
                            const void* key, const void* value, void* key_cache, void* value_cache,
                            const int32_t* block_indices) {
    if (q_dtype == DT_F16) {
        if (kv_dtype == DT_U8) return launch_epl<DT_F16, DT_U8>(s, st, sh, key, value, key_cache, value_cache, block_indices);
        if (kv_dtype == DT_F16) return launch_epl<DT_F16, DT_F16>(s, st, sh, key, value, key_cache, value_cache, block_indices);
        return launch_epl<DT_F16, DT_BF16>(s, st, sh, key, value, key_cache, value_cache, block_indices);
    }
    if (kv_dtype == DT_U8) return launch_epl<DT_BF16, DT_U8>(s, st, sh, key, value, key_cache, value_cache, block_indices);
    if (kv_dtype == DT_F16) return launch_epl<DT_BF16, DT_F16>(s, st, sh, key, value, key_cache, value_cache, block_indices);
    return launch_epl<DT_BF16, DT_BF16>(s, st, sh, key, value, key_cache, value_cache, block_indices);
}

}  // namespace pa
