// Chunked-prefill (and mixed prefill + decode) PagedAttention on the gfx950 matrix cores, over a 16-bit
// KV cache (f16 or bf16, same type as the query) or a u8 cache.  u8 codes are staged in LDS zero-extended
// to 16 bits -- read as f16 that is the subnormal code * 2^-24, which the matrix cores multiply exactly --
// and the rows' scale / zero-point are applied to the accumulator tiles:
//   logit = scale * sc_k * (q . codes - zp_k * sum(q))
//   out   = sum_t w_t codes_t - sum_t w_t zp_v,   w_t = p_t * sc_v  (the same f16-rounded w_t on both sides)
//
// Work item = (sequence, tile of QT query tokens, range of KV blocks, kv head): one workgroup of 512
// or 256 threads.  The query rows of the tile are the (token, head-in-group) pairs that share the kv head
// -- up to 128 rows, 16 or 32 per wave -- so a KV block fetched once serves the whole
// GQA group and QT tokens.  Long contexts are cut into ranges of KV blocks (split-K) so that work
// items stay comparable in length; their partial (max, denominator, accumulator) rows are merged
// by a second kernel.
// KV blocks (32 tokens) travel global -> registers (two or three blocks in flight per thread) -> LDS (two K
// slots, four V slots, one barrier per block), or straight into LDS; K rows are read back as MFMA A operands with
// ds_read_b128, V rows through the LDS transpose read (ds_read_b64_tr_b16), which hands each lane
// four consecutive tokens of one channel.  A block is worked through in one go: QK, softmax, rescale, PV.
//   S^T[token][row] = K . Q^T          v_mfma_f32_16x16x32_{f16,bf16}
//   O^T[d][row]    += V^T . P^T        P (u8 caches: P times the V row's scale) in the operand type as hi + lo
//                                      halves; one half alone (8 bits for bf16, 11 for f16) leaves outputs outside
//                                      the tolerance when large V elements of opposite sign cancel
// Causal mask: row of token i (global position past + i) sees positions <= past + i, and with a
// sliding window only the last `sliding_window` of them.  Online softmax in the log2 domain.
// Block-sparse sequences (XATT variant): a row additionally sees only the key blocks its (head, query block) kept
// (one bit per key block, see pa_xattention.hip), and the work item walks a list of the KV blocks that some row of
// it kept instead of its whole range.
//
// Roofline: dense MFMA.  Flops per (query row, visible position): 4 * D.
#include "pa_device.h"

#include <climits>
#include <type_traits>

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
constexpr float LN2 = 0.6931471805599453f;

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

// Reductions over the four 16-lane groups of a wave with the gfx950 lane-swap instructions (no LDS round trip):
// v_permlane16_swap exchanges the odd 16-lane rows of its first operand with the even rows of the second,
// v_permlane32_swap the upper half of the first with the lower half of the second.  With both operands holding
// the same value the pair afterwards holds, per lane, the values of the two rows (halves) being combined.
__device__ __forceinline__ void swap_rows16(float& a, float& b) {
    asm volatile("s_nop 1\n\tv_permlane16_swap_b32 %0, %1\n\ts_nop 1" : "+v"(a), "+v"(b));
}
__device__ __forceinline__ void swap_halves32(float& a, float& b) {
    asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1\n\ts_nop 1" : "+v"(a), "+v"(b));
}
// (the maxima as instructions of their own: behind the lane swaps the compiler no longer knows its operands to be
// ordinary numbers and puts a quieting `v_max x, x, x` in front of every fmaxf)
__device__ __forceinline__ float max_raw(float a, float b) {
    float r;
    asm("v_max_f32 %0, %1, %2" : "=v"(r) : "v"(a), "v"(b));
    return r;
}
__device__ __forceinline__ float xor_max_g(float v) {
    float a = v, b = v;
    swap_rows16(a, b);
    a = b = max_raw(a, b);
    swap_halves32(a, b);
    return max_raw(a, b);
}
__device__ __forceinline__ float xor_sum_g(float v) {
    float a = v, b = v;
    swap_rows16(a, b);
    a = b = a + b;
    swap_halves32(a, b);
    return a + b;
}

// acc + the two 16-bit floats of `w` (one instruction: a dot product with (1, 1))
template <int DT>
__device__ __forceinline__ float add_pair(uint32_t w, float acc) {
    if (DT == DT_F16) {
        typedef _Float16 h2 __attribute__((ext_vector_type(2)));
        return __builtin_amdgcn_fdot2(__builtin_bit_cast(h2, w), __builtin_bit_cast(h2, 0x3c003c00u), acc, false);
    }
    typedef __bf16 b2 __attribute__((ext_vector_type(2)));
    return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(b2, w), __builtin_bit_cast(b2, 0x3f803f80u), acc, false);
}

// f32 -> cache-type bits, two values at a time
template <int DT>
__device__ __forceinline__ uint32_t pack2(float a, float b) {
    if (DT == DT_F16) {
        typedef _Float16 h2 __attribute__((ext_vector_type(2)));
        return __builtin_bit_cast(uint32_t, h2{(_Float16)a, (_Float16)b});
    }
    typedef __bf16 b2 __attribute__((ext_vector_type(2)));
    return __builtin_bit_cast(uint32_t, b2{(__bf16)a, (__bf16)b});
}

// ---- KV block fetches -------------------------------------------------------------------------------------
// Through registers (u8 caches, whose rows are transformed on the way to LDS; block-sparse items; head size 64):
// ordinary loads into three register sets, three blocks in flight per thread; the compiler counts the outstanding
// loads itself (it waits for the oldest set only).  Every step issues the same loads per thread: tile indices are
// clamped rather than skipped.
typedef uint32_t u2v __attribute__((ext_vector_type(2)));
template <bool U8>
struct KvRegs;
template <>
struct KvRegs<false> {
    static constexpr int LOADS = 2;
    u4v k, v;  // one 16-byte chunk of the K block and of the V block
};
template <>
struct KvRegs<true> {
    static constexpr int LOADS = 4;
    u2v kc, kh, vc, vh;  // 8 codes and the row header (scale, zero-point) of a K row and of a V row
};
__device__ __forceinline__ void kv_issue(KvRegs<false>& r, const uint8_t* kp, const uint8_t* vp) {
    r.k = *reinterpret_cast<const u4v*>(kp);
    r.v = *reinterpret_cast<const u4v*>(vp);
}
__device__ __forceinline__ void kv_issue(KvRegs<true>& r, const uint8_t* krow, const uint8_t* vrow, int code_off) {
    r.kc = *reinterpret_cast<const u2v*>(krow + code_off);
    r.kh = *reinterpret_cast<const u2v*>(krow);
    r.vc = *reinterpret_cast<const u2v*>(vrow + code_off);
    r.vh = *reinterpret_cast<const u2v*>(vrow);
}

// Straight into LDS (dense items over 16-bit caches, head size 128): one instruction moves 64 x 16 bytes from
// per-lane global addresses to 1024 consecutive bytes of LDS at a wave-uniform address; no registers, no LDS stores.
__device__ __forceinline__ void dma16(const uint8_t* src, uint8_t* lds_dst) {
    typedef __attribute__((address_space(3))) void* lds_p;
    typedef const __attribute__((address_space(1))) void* glb_p;
    __builtin_amdgcn_global_load_lds((glb_p)src, (lds_p)lds_dst, 16, 0, 0);
}
// Waits until at most N of the wave's vector-memory operations are outstanding (gfx9 encoding: vmcnt in bits 3:0 and
// 15:14; the other counters left at their maxima).
// Workgroup barrier for LDS traffic only.  __syncthreads() (and a workgroup fence of any kind) makes the compiler wait
// for every copy into LDS that is in flight, the prefetched blocks included; here the wave waits for its own LDS
// operations, meets the others, and the copies it must have finished are named by the caller (wait_vmem).  The
// barrier instruction and the empty asm statements keep the compiler from moving LDS accesses across.
__device__ __forceinline__ void lds_barrier() {
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0); vmcnt and expcnt at their maxima
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
}
template <int N>
__device__ __forceinline__ void wait_vmem() {
    __builtin_amdgcn_s_waitcnt((N & 0xf) | ((N >> 4) << 14) | 0x0f70);
}

// DT: type of the MFMA operands and of the rows staged in LDS; QDT: type of query and output; U8: the cache holds
// `f32 scale | f32 zero-point | D codes` rows; codes go to LDS as 16-bit words, headers to a small table beside them.
// NG: 16-row groups per wave.  1 = up to 128 query rows per 512-thread workgroup, the variant for mixed steps over
// 16-bit caches and for work items with few rows (single-token sequences: G rows), where a second group would only cost
// arithmetic; it fits four waves per SIMD over 16-bit caches.  2 = 32 rows per wave (the 256-thread variants below).
// A block is worked through in one go: QK, softmax, rescale, PV.
// XATT: the work items belong to block-sparse sequences.
// HALF: 256-thread workgroups of 128 rows whose KV blocks go through registers, two load units per thread (u8 caches,
// whose codes are widened on the way to LDS): two such workgroups share a CU and fill in for each other at the
// barriers.  (One 512-thread workgroup of 256 rows per CU, with a three-block software pipeline inside each wave, took
// 0.296 ms for what this variant does in 0.255 ms: a third of the launch had neither pipe busy.)
// DMA: 256-thread workgroups whose KV blocks go straight from global memory into LDS (four K and four V slots, three
// blocks in flight behind the one being worked on).  Rows sit in LDS unpadded; instead the 16-byte pieces of a row are
// permuted: K row r keeps piece p at position p ^ (r & 15) (16 lanes read one piece of 16 rows), V row r at
// p ^ 2 (r & 7) (the transpose read takes 32 bytes of each of four consecutive rows), which keeps both operand reads
// free of bank conflicts -- the permutation is applied on the global side of the copy, each lane fetching the piece
// that belongs at its LDS position.  With no
// staging registers the kernel fits three waves per SIMD at two 16-row groups per wave: half the LDS operand traffic
// per matrix instruction of the one-group variant.
template <int D, int DT, int QDT, bool U8, int NG, bool XATT, bool DMA, bool HALF = false>
__global__ __launch_bounds__((DMA || HALF) ? 256 : 512, D > 128 ? 1 : (DMA || HALF) ? 2 : U8 ? 2 : (XATT && DT == DT_F16 && D == 128) ? 3 : 4)
void pa_prefill16_kernel(PrefillArgs a) {
    static_assert(!U8 || DT == DT_F16, "u8 codes are multiplied as f16");
    static_assert(U8 || DT == QDT, "16-bit caches are used in the query's type");
    static_assert(!DMA || (!U8 && !XATT && D == 128), "the straight-to-LDS variant: dense items, 16-bit caches, head size 128");
    static_assert(!(DMA && HALF) && (!HALF || (NG == 2 && !XATT)), "the register variant of 256 threads: dense items, two row groups per wave");
    constexpr int NT = (DMA || HALF) ? 256 : 512;
    constexpr int NCH = TOK * (D * 2 / 16);  // 16-byte chunks (eight codes of a u8 row) per block and tensor: 512 (D = 128) or 256 (D = 64)
    constexpr int UPT = (NCH + NT - 1) / NT;  // load units (a chunk, or eight codes and a row header) per thread and tensor
    constexpr int ROWB = D * 2;            // bytes of a row as staged in LDS
    constexpr int CROWB = U8 ? D + 8 : D * 2;  // bytes of a row in the cache
    constexpr int LROWK = DMA ? ROWB : ROWB + 16;  // LDS row strides chosen so that the operand reads are bank-conflict free:
    constexpr int LROWV = DMA ? ROWB : ROWB + 32;  // K rows are read 16 B per lane, V rows 32 B per 4 lanes (transpose read)
    constexpr int TILEK = TOK * LROWK, TILEV = TOK * LROWV;
    constexpr int NKS = DMA ? 4 : 2, NVS = 4;  // K and V slots
    constexpr int KS = D / 32;
    constexpr int RT = D / 16;
    constexpr int CPR = ROWB / 16;         // 16-byte chunks per row
    static_assert(DMA || NCH <= NT * UPT, "one chunk per load unit");
    constexpr int HDRB = U8 ? 4 * TOK * 4 : 0;  // per buffer: sc_k | zp_k * sc_k | sc_v | zp_v, one f32 per token each
    constexpr float CODE_UNIT = 16777216.0f;    // a code byte read as f16 is code * 2^-24
    // Block t+1 is read while block t+2 is written: two K slots; the V and header slots are indexed modulo four.
    constexpr int OFF_V = NKS * TILEK, OFF_H = NKS * TILEK + NVS * TILEV;
    __shared__ __align__(16) uint8_t smem[DMA ? 16 : NKS * TILEK + NVS * TILEV + 4 * HDRB];  // K slots | V slots | headers[4]
    // DMA: every slot is an LDS object of its own, so that the compiler can tell a copy into one slot from the operand
    // reads of another (it orders reads after the copies that may have written what they read; with one array for all
    // slots that would be every copy in flight, the prefetched blocks included)
    __shared__ __align__(16) uint8_t dk0[DMA ? TILEK : 16], dk1[DMA ? TILEK : 16], dk2[DMA ? TILEK : 16], dk3[DMA ? TILEK : 16];
    __shared__ __align__(16) uint8_t dv0[DMA ? TILEV : 16], dv1[DMA ? TILEV : 16], dv2[DMA ? TILEV : 16], dv3[DMA ? TILEV : 16];
    auto kslot = [](int j) { return (j & 1); };
    auto vslot = [](int j) { return (j & (NVS - 1)); };

    const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
    const int n = lane & 15, g = lane >> 4;
    const StepDev& st = a.st;
    const int Hq = a.sh.Hq, Hkv = a.sh.Hkv, G = a.G;
    const int hkv = blockIdx.x % Hkv;
    const PrefillItem item = a.items[blockIdx.x / Hkv];
    const int b = item.b;
    const int t0 = st.subsequence_begins[b];
    const int past = st.past_lens[b];
    const int q0 = item.q0;
    const int R = item.nq * G;  // query rows of this tile
    const int tb = item.tb, te = item.te;
    // the KV blocks this workgroup walks: all of [tb, te), or (block-sparse) those listed for (item, kv head); the
    // list is read through the scalar path (uniform index)
    typedef const int32_t __attribute__((address_space(4))) * const_i32_ptr;
    typedef const uint32_t __attribute__((address_space(4))) * const_u32_ptr;
    const const_i32_ptr tile_list =
        XATT ? (const_i32_ptr)(uintptr_t)(a.xatt.item_tiles + (long)blockIdx.x * a.xatt.tiles_stride) : (const_i32_ptr)0;
    const int cnt = XATT ? tile_list[0] : te - tb;
    auto tile_at = [&](int j) __attribute__((always_inline)) {  // j-th block of the walk (j beyond the end: the last one)
        if constexpr (XATT) return tb + tile_list[1 + max(min(j, cnt - 1), 0)];
        else return min(tb + j, te - 1);
    };
    // the block table is read through the constant address space: uniform index, so a scalar load, which does not
    // share a counter with the KV fetches in flight
    const const_i32_ptr table = (const_i32_ptr)(uintptr_t)(a.block_indices + st.block_indices_begins[b]);
    const int sw = st.sliding_window;

    // this wave's two 16-row groups
    int row_pos[2];    // global position of the row's token (-1: no such row)
    int row_id[2];     // token * Hq + head (the host refuses steps with 2^31 rows or more)
    s8v qreg[2][KS];
    // block-sparse: bit k of a row's four words in LDS = the row kept key block kb_lo + k (an item walks at most 128
    // KV blocks).  In LDS because the word is picked by a run-time index, which would put a register array in scratch.
    __shared__ uint32_t row_keep[XATT ? 256 * 4 : 1];
    const int xt_shift = XATT ? a.xatt.xb_shift - 5 : 0;  // KV blocks per key block, as a shift
    const int kb_lo = XATT ? tb >> xt_shift : 0;
#pragma unroll
    for (int gi = 0; gi < NG; ++gi) {
        // rows beyond R repeat the tile's last row (no branch around the loads); nothing of theirs is stored
        const bool ok = 16 * NG * wv + 16 * gi + n < R;
        const int rho = min(16 * NG * wv + 16 * gi + n, R - 1);
        const int qtok = q0 + rho / G;
        row_pos[gi] = ok ? past + qtok : -1;
        row_id[gi] = (t0 + qtok) * Hq + hkv * G + rho % G;
        if constexpr (XATT) {
            const XattSeq* xs = a.xatt.seqs + a.xatt.seq_of[b];
            const int words = xs->words;
            const uint32_t* mrow = a.xatt.mask + xs->mask_off +
                                   ((long)(hkv * G + rho % G) * xs->nqb + (((past + qtok) >> a.xatt.xb_shift) - xs->qb0)) * words;
            const int w0 = kb_lo >> 5, sh = kb_lo & 31;
            // words past the row's end are never looked at
            const uint32_t wa = mrow[min(w0, words - 1)], wb = mrow[min(w0 + 1, words - 1)], wc = mrow[min(w0 + 2, words - 1)],
                           wd = mrow[min(w0 + 3, words - 1)], we = mrow[min(w0 + 4, words - 1)];
            // the wave's own rows: written and read by the same lanes group (row 16 * (NG * wv + gi) + n, all four g alike)
            *reinterpret_cast<u4v*>(row_keep + 4 * (16 * NG * wv + 16 * gi + n)) =
                u4v{(uint32_t)((((uint64_t)wb << 32) | wa) >> sh), (uint32_t)((((uint64_t)wc << 32) | wb) >> sh),
                    (uint32_t)((((uint64_t)wd << 32) | wc) >> sh), (uint32_t)((((uint64_t)we << 32) | wd) >> sh)};
        }
#pragma unroll
        for (int s = 0; s < KS; ++s) {
            u4v v = *reinterpret_cast<const u4v*>(a.query + (long)row_id[gi] * D + 32 * s + 8 * g);
            if (QDT != DT) {  // bf16 query against f16 operands
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    v[e] = pack2<DT_F16>(__builtin_bit_cast(float, v[e] << 16), __builtin_bit_cast(float, v[e] & 0xffff0000u));
            }
            qreg[gi][s] = __builtin_bit_cast(s8v, v);
        }
    }
    const float scl = st.scale * LOG2E;
    float qsum[2] = {0.0f, 0.0f};  // u8: sum of the row's query elements (for the zero-point term), times scl
    if (U8) {
#pragma unroll
        for (int gi = 0; gi < NG; ++gi) {
            float part = 0.0f;
#pragma unroll
            for (int s = 0; s < KS; ++s) {
                const h8 qh = __builtin_bit_cast(h8, qreg[gi][s]);
#pragma unroll
                for (int e = 0; e < 8; ++e) part += (float)qh[e];
            }
            qsum[gi] = xor_sum_g(part) * scl;
        }
    }
    // positions every row of this wave can see: blocks inside [free_lo, free_hi] need no mask
    int free_hi, free_lo;
    {
        // rows that do not exist (beyond R) are left out: what they compute is never stored
        int lim = INT_MAX, low = INT_MIN;
#pragma unroll
        for (int gi = 0; gi < NG; ++gi) {
            lim = min(lim, row_pos[gi] < 0 ? INT_MAX : row_pos[gi]);
            low = max(low, row_pos[gi] + 1 - sw);  // largest window start
        }
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) {
            lim = min(lim, __shfl_xor(lim, o, WAVE));
            low = max(low, __shfl_xor(low, o, WAVE));
        }
        free_hi = lim;
        free_lo = sw > 0 ? max(low, 0) : 0;
    }

    float m_run[2] = {-INFINITY, -INFINITY}, l_part[2] = {0.0f, 0.0f};
    // 16-bit caches keep the running maximum negated (NO_MAX while the row has seen nothing), ready for the exponent's
    // multiply-add, and the level (log2, relative to the running maximum) a block's largest probability must stay
    // under for the block to do without the second, low-half product: log2(LO_SHARE x the row's denominator when
    // last looked at).
    constexpr float NO_MAX = 1e30f;
    float neg_m[2] = {NO_MAX, NO_MAX}, lo_at[2] = {-INFINITY, -INFINITY};
    float zsum[2] = {0.0f, 0.0f};  // u8: this lane's share of sum_t w_t zp_v
    f4 acc[2][RT];
#pragma unroll
    for (int gi = 0; gi < NG; ++gi)
#pragma unroll
        for (int r = 0; r < RT; ++r) acc[gi][r] = f4{0.0f, 0.0f, 0.0f, 0.0f};

    // three blocks in flight in registers.  16-bit cache: thread = one 16-byte chunk of K and of V per block.
    // u8 cache: thread = (row, group of 8 codes) plus the row's header; it writes the 8 codes as 16-bit words (16
    // bytes) -- same LDS address either way.  Threads beyond the chunk count repeat the loads of the first ones.
    KvRegs<U8> set[HALF ? 2 : 3][UPT];
    const bool loader = tid < NCH;
    const int ltid = tid % NCH;
    const int lds_k = (ltid / CPR) * LROWK + (ltid % CPR) * 16;
    const int lds_v = OFF_V + (ltid / CPR) * LROWV + (ltid % CPR) * 16;
    // (a thread's second load unit, where it has one: the chunk NT further on, i.e. the same piece of the row 16 below)
    auto unit_loads = [&](int uu) __attribute__((always_inline)) { return uu == 0 ? loader : tid + NT * uu < NCH; };
    auto unit_id = [&](int uu) __attribute__((always_inline)) { return uu == 0 ? ltid : (tid + NT * uu) % NCH; };
    auto unit_lds_k = [&](int uu) __attribute__((always_inline)) { return uu == 0 ? lds_k : (unit_id(uu) / CPR) * LROWK + (unit_id(uu) % CPR) * 16; };
    auto unit_lds_v = [&](int uu) __attribute__((always_inline)) { return uu == 0 ? lds_v : OFF_V + (unit_id(uu) / CPR) * LROWV + (unit_id(uu) % CPR) * 16; };
    const int kv_len = past + st.subsequence_begins[b + 1] - t0;
    // The kernel's tiles are 32 tokens: one 32-token cache block, or two 16-token blocks, in which case each row is
    // fetched from the block it lies in (a last tile of one block repeats it; those rows lie beyond kv_len).
    // tile_base(tile, upper): what to add to `row * CROWB` for a row of the tile's lower or upper half.
    const bool bs16 = a.sh.bs == 16;
    const int sub_mask = bs16 ? 0 : (a.sh.bs >> 5) - 1, sub_shift = bs16 ? 0 : 31 - __builtin_clz(a.sh.bs >> 5);
    const int last_block16 = (kv_len - 1) >> 4;
    auto tile_base = [&](int tile, bool upper) __attribute__((always_inline)) -> long {
        // (blocks of 32 tokens or more, a power of two: the tile is one 32-token part of its block)
        if (!bs16) return ((long)table[tile >> sub_shift] * Hkv + hkv) * ((long)a.sh.bs * CROWB) + (long)(tile & sub_mask) * (TOK * CROWB);
        const long lo = ((long)table[2 * tile] * Hkv + hkv) * (16 * CROWB);
        const long hi = ((long)table[min(2 * tile + 1, last_block16)] * Hkv + hkv) * (16 * CROWB) - 16 * CROWB;
        return upper ? hi : lo;
    };
    auto fetch = [&](KvRegs<U8> (&rs)[UPT], int j) __attribute__((always_inline)) {
#pragma unroll
        for (int uu = 0; uu < UPT; ++uu) {
            KvRegs<U8>& r = rs[uu];
            const int lt = unit_id(uu);
            const long blk = tile_base(tile_at(j), lt / CPR >= 16);
            if constexpr (U8) {
                const long row = blk + (long)(lt / CPR) * CROWB;
                kv_issue(r, a.key_cache + row, a.value_cache + row, 8 + (lt % CPR) * 8);
            } else {
                kv_issue(r, a.key_cache + blk + (long)lt * 16, a.value_cache + blk + (long)lt * 16);
            }
        }
    };
    // rows beyond the sequence's tokens (the tail of its last block) may hold anything: their K columns are masked
    // by the causal select, their V rows are cleared here so that 0 * garbage cannot reach the accumulators
    // j = block number within the item's range; it selects the LDS slots
    auto stash = [&](KvRegs<U8> (&rs)[UPT], int j) __attribute__((always_inline)) {
        const int tile = tile_at(j);
#pragma unroll
        for (int uu = 0; uu < UPT; ++uu) {
        KvRegs<U8>& r = rs[uu];
        const int lt = unit_id(uu);
        if (unit_loads(uu) && j < cnt) {
            const bool live = tile * TOK + lt / CPR < kv_len;
            uint8_t* kd = smem + kslot(j) * TILEK + unit_lds_k(uu);
            uint8_t* vd = smem + vslot(j) * TILEV + unit_lds_v(uu);
            if constexpr (U8) {
                // Codes go to LDS as 16-bit words holding (code - c) * 2^-24, c the integer nearest the row's
                // zero-point: an exact f16 subnormal either way, but the sums the matrix pipe forms stay near the
                // size of the result instead of riding on sum(w * zp).  That matters because the pipe adds every
                // product into its accumulator with truncation at the accumulator's last bit: a row that leans on
                // an early token and then adds thousands of small products loses about half a unit in the last
                // place of the accumulator per product, and with plain codes that accumulator is several times the
                // size of the output.
                typedef _Float16 h2 __attribute__((ext_vector_type(2)));
                const uint32_t k0 = r.kc[0], k1 = r.kc[1], v0 = r.vc[0], v1 = r.vc[1];
                const uint32_t ksb = r.kh[0], kzb = r.kh[1], vsb = r.vh[0], vzb = r.vh[1];  // (a bit cast straight from a vector element reads element 0)
                const float kzf = __builtin_bit_cast(float, kzb), vzf = __builtin_bit_cast(float, vzb);
                const float kc = rintf(fminf(fmaxf(kzf, 0.0f), 255.0f)), vc = rintf(fminf(fmaxf(vzf, 0.0f), 255.0f));
                const h2 kneg = __builtin_bit_cast(h2, 0x80008000u | ((uint32_t)kc * 0x00010001u));  // -c * 2^-24, twice
                const h2 vneg = __builtin_bit_cast(h2, 0x80008000u | ((uint32_t)vc * 0x00010001u));
                auto centred = [](uint32_t word, h2 neg) {
                    return __builtin_bit_cast(uint32_t, __builtin_bit_cast(h2, word) + neg);  // exact: integers times 2^-24
                };
                *reinterpret_cast<u4v*>(kd) = u4v{centred(__builtin_amdgcn_perm(0u, k0, 0x0c010c00u), kneg),
                                                  centred(__builtin_amdgcn_perm(0u, k0, 0x0c030c02u), kneg),
                                                  centred(__builtin_amdgcn_perm(0u, k1, 0x0c010c00u), kneg),
                                                  centred(__builtin_amdgcn_perm(0u, k1, 0x0c030c02u), kneg)};
                *reinterpret_cast<u4v*>(vd) = u4v{centred(__builtin_amdgcn_perm(0u, v0, 0x0c010c00u), vneg),
                                                  centred(__builtin_amdgcn_perm(0u, v0, 0x0c030c02u), vneg),
                                                  centred(__builtin_amdgcn_perm(0u, v1, 0x0c010c00u), vneg),
                                                  centred(__builtin_amdgcn_perm(0u, v1, 0x0c030c02u), vneg)};
                if (lt % CPR == 0) {  // the table holds what is left of the zero-points
                    float* hdr = reinterpret_cast<float*>(smem + OFF_H + (j & 3) * HDRB) + lt / CPR;
                    const float sck = __builtin_bit_cast(float, ksb);
                    hdr[0] = live ? sck : 0.0f;
                    hdr[TOK] = live ? (kzf - kc) * sck : 0.0f;
                    hdr[2 * TOK] = live ? __builtin_bit_cast(float, vsb) : 0.0f;
                    hdr[3 * TOK] = live ? vzf - vc : 0.0f;
                }
            } else {
                *reinterpret_cast<u4v*>(kd) = r.k;
                *reinterpret_cast<u4v*>(vd) = live ? r.v : u4v{0u, 0u, 0u, 0u};
            }
        }
        }
    };
    const bool active = 16 * NG * wv < R;  // waves without rows only help moving blocks
    // A single-token sequence whose scores are wanted: wave 0 keeps its heads' probabilities and per-tile maxima in LDS
    // and the workgroup writes them out behind the loop.  (A store inside the loop would make every wait for a block
    // fetch a wait for all of them: loads and stores share a counter and complete out of order with respect to each
    // other.)  The host keeps such items at single_item_max_tiles(G) tiles.
    constexpr bool STASH = !U8 && !XATT && !DMA && NG == 1;
    __shared__ __align__(16) uint8_t pkeep[STASH ? SINGLE_STASH_BYTES : 16];
    bool emit = false;
    if constexpr (STASH) emit = a.p_out != nullptr && a.single_idx[b] >= 0;

    // ---- the pieces of work on a block ---------------------------------------------------------------------
    // S^T = K . Q^T for both row groups (block number jk) and O^T += V^T . P^T (block number jv), issued as one
    // stream.  A matrix instruction's result is ready about eight issue slots later, so instructions that feed each
    // other are kept at least that far apart: per 32-channel slice s the stream is
    //     4 x QK (the four S accumulators) | 4 x PV (output tiles 2s, 2s+1, both row groups)
    //                                      | 4 x PV with the low halves of P for the tiles of slice s-1 (16-bit caches)
    // V operands come through the LDS transpose read: source lane (e = n >> 2, q = n & 3) of a 16-lane group
    // supplies 4 channels of token 16 h + 4 g + e; lane n receives channel 16 r + n of tokens 16 h + 4 g + 0..3.
    auto load_v = [&](const uint8_t* vb, int r) __attribute__((always_inline)) {
        const uint8_t* p0 = DMA ? vb + (4 * g + (n >> 2)) * LROWV + (((2 * r + ((n & 3) >> 1)) ^ (((4 * g + (n >> 2)) & 7) << 1)) << 4) + 8 * (n & 1)
                                : vb + (4 * g + (n >> 2)) * LROWV + (16 * r + 4 * (n & 3)) * 2;
        const s4v v0 = lds_read_tr16(p0);
        const s4v v1 = lds_read_tr16(p0 + 16 * LROWV);
        return s8v{v0[0], v0[1], v0[2], v0[3], v1[0], v1[1], v1[2], v1[3]};
    };
    auto qk_pv_at = [&](bool do_qk, const uint8_t* kb, f4 (&sc)[2][2], bool do_pv, const uint8_t* vb, const u4v (&pb)[2],
                        const u4v (&pl)[2]) __attribute__((always_inline)) {
        if (do_qk) {
#pragma unroll
            for (int gi = 0; gi < NG; ++gi) sc[gi][0] = sc[gi][1] = f4{0.0f, 0.0f, 0.0f, 0.0f};
        }
        s8v vprev[2];
#pragma unroll
        for (int s = 0; s <= KS; ++s) {
            if (do_qk && s < KS) {
#pragma unroll
                for (int u = 0; u < 2; ++u) {
                    const s8v kop = DMA ? *reinterpret_cast<const s8v*>(kb + (16 * u + n) * LROWK + (((4 * s + g) ^ n) << 4))
                                        : *reinterpret_cast<const s8v*>(kb + (16 * u + n) * LROWK + (32 * s + 8 * g) * 2);
#pragma unroll
                    for (int gi = 0; gi < NG; ++gi) sc[gi][u] = mma<DT>(kop, qreg[gi][s], sc[gi][u]);
                }
            }
            if (do_pv) {
                s8v vcur[2];
                if (s < KS) {
#pragma unroll
                    for (int h = 0; h < 2; ++h) {
                        vcur[h] = load_v(vb, 2 * s + h);
#pragma unroll
                        for (int gi = 0; gi < NG; ++gi)
                            acc[gi][2 * s + h] = mma<DT>(vcur[h], __builtin_bit_cast(s8v, pb[gi]), acc[gi][2 * s + h]);
                    }
                }
                if (s > 0) {  // the low halves of P, one slice behind
#pragma unroll
                    for (int h = 0; h < 2; ++h) {
#pragma unroll
                        for (int gi = 0; gi < NG; ++gi)
                            acc[gi][2 * s - 2 + h] =
                                mma<DT>(vprev[h], __builtin_bit_cast(s8v, pl[gi]), acc[gi][2 * s - 2 + h]);
                    }
                }
                vprev[0] = vcur[0];
                vprev[1] = vcur[1];
            }
        }
    };
    // u8 caches: masks + online softmax of block `tile` (number j): weights as MFMA operands, rescale factors.
    // The running maximum is only raised when a block exceeds it by more than 2^4: probabilities then stay
    // below 16 and the accumulators are rescaled a few times per row instead of once per block.
    auto softmax = [&](auto masked_c, const f4 (&sc)[2][2], int tile, int j, u4v (&pb)[2], u4v (&pl)[2],
                       float (&corr)[2], const bool (&kept)[2]) __attribute__((always_inline)) {
        constexpr bool MASKED = decltype(masked_c)::value;
        const int pos0 = tile * TOK + 4 * g;
        f4 h_sck[2], h_zpk[2], h_scv[2], h_zpv[2];  // headers of this lane's 8 tokens (16 u + 4 g + i)
        if (U8) {
            const float* hdr = reinterpret_cast<const float*>(smem + OFF_H + (j & 3) * HDRB);
#pragma unroll
            for (int u = 0; u < 2; ++u) {
                h_sck[u] = *reinterpret_cast<const f4*>(hdr + 16 * u + 4 * g);
                h_zpk[u] = *reinterpret_cast<const f4*>(hdr + TOK + 16 * u + 4 * g);
                h_scv[u] = *reinterpret_cast<const f4*>(hdr + 2 * TOK + 16 * u + 4 * g);
                h_zpv[u] = *reinterpret_cast<const f4*>(hdr + 3 * TOK + 16 * u + 4 * g);
            }
        }
#pragma unroll
        for (int gi = 0; gi < NG; ++gi) {
            float x[8];
            float mx = -INFINITY;
            if (U8) {
#pragma unroll
                for (int u = 0; u < 2; ++u)
#pragma unroll
                    for (int i = 0; i < 4; ++i)
                        x[4 * u + i] = fmaf(sc[gi][u][i] * (scl * CODE_UNIT), h_sck[u][i], -h_zpk[u][i] * qsum[gi]);
            }
            if (MASKED) {
                const int lim = row_pos[gi];
                const int low = sw > 0 ? max(0, lim + 1 - sw) : 0;
#pragma unroll
                for (int jj = 0; jj < 8; ++jj) {
                    const int pos = pos0 + 16 * (jj >> 2) + (jj & 3);
                    x[jj] = (pos <= lim && pos >= low && kept[gi]) ? x[jj] : -INFINITY;
                }
            }
#pragma unroll
            for (int jj = 0; jj < 8; ++jj) mx = fmaxf(mx, x[jj]);
            mx = xor_max_g(mx);
            const float m_new = mx > m_run[gi] + 4.0f ? mx : m_run[gi];
            const float m_safe = m_new == -INFINITY ? 0.0f : m_new;
            corr[gi] = __builtin_amdgcn_exp2f(m_run[gi] - m_safe);
            float p[8];
            float psum = 0.0f;
#pragma unroll
            for (int jj = 0; jj < 8; ++jj) {
                p[jj] = __builtin_amdgcn_exp2f(x[jj] - m_safe);
                psum += p[jj];
            }
            if (U8) {
                // Weights carry the V row's scale.  They go to the matrix pipe as an f16 value plus what that
                // rounding dropped (a second f16), like the probabilities of the 16-bit caches: with 11 bits alone
                // a row that leans on a few tokens with large, opposite V values misses the tolerance now and then.
                // The zero-point term takes the f32 weight, which the two halves reproduce to 2^-23.
                float zs = 0.0f;
#pragma unroll
                for (int jj = 0; jj < 4; ++jj) {
                    typedef _Float16 h2 __attribute__((ext_vector_type(2)));
                    const float w0 = p[2 * jj] * h_scv[jj >> 1][(2 * jj) & 3];
                    const float w1 = p[2 * jj + 1] * h_scv[jj >> 1][(2 * jj + 1) & 3];
                    uint32_t wb = __builtin_bit_cast(uint32_t, h2{(_Float16)w0, (_Float16)w1});
                    // one rounded value for both uses below: left alone, the compiler forms the f16 weight twice, once
                    // from the f32 product (two roundings) and once with a mixed-precision multiply (one rounding); at
                    // a tie the two differ by one f16 step, and the low half would belong to another high half
                    asm volatile("" : "+v"(wb));
                    pb[gi][jj] = wb;
                    const h2 hi = __builtin_bit_cast(h2, wb);
                    pl[gi][jj] = __builtin_bit_cast(uint32_t, h2{(_Float16)(w0 - (float)hi[0]), (_Float16)(w1 - (float)hi[1])});
                    zs = fmaf(w0, h_zpv[jj >> 1][(2 * jj) & 3], zs);
                    zs = fmaf(w1, h_zpv[jj >> 1][(2 * jj + 1) & 3], zs);
                }
                zsum[gi] = zsum[gi] * corr[gi] + zs;
            }
            l_part[gi] = l_part[gi] * corr[gi] + psum;
            m_run[gi] = m_new;
        }
    };

    // ---- 16-bit caches: the softmax of a block, and the product with the probabilities --------------------------
    // Probabilities enter the matrix pipe rounded to the cache type, as a high half and -- what that rounding dropped --
    // a low half: 16 significant bits for bf16, 22 for f16.  With the high half alone (8 bits for bf16) the rounding
    // of a single dominant token's probability is outside the tolerance whenever large V values of opposite sign
    // cancel.  The denominator is the sum of the rounded halves (one dot-product instruction per pair), so a row's
    // weights stay a convex combination whatever the rounding did.
    // f16 caches: 11 bits are enough for every token that is a small share of its row, so the low halves follow only
    // for blocks in which some row has a token whose probability exceeds 2^LO_SHARE_LOG2 of that row's denominator so
    // far (the running one, a lower bound of the final one).  The rounding errors of the tokens below that share add
    // up like noise of at most 2^-12 sqrt(share) x the spread of V per row; a row that leans on a few tokens -- where
    // one rounding error is the whole error -- takes both halves.  bf16 caches always take both: at 8 bits the share
    // would have to be so small that nearly every block of a context of a few thousand tokens exceeds it.
    // Returns (wave-uniform) whether this block needs the low halves.
    constexpr bool LO_ALWAYS = DT == DT_BF16;
    constexpr float LO_SHARE_LOG2 = -2.0f;
    auto softmax16 = [&](auto masked_c, const f4 (&sc)[2][2], int tile, int j, u4v (&pb)[2], float (&p)[2][8],
                         const bool (&kept)[2]) __attribute__((always_inline)) -> bool {
        constexpr bool MASKED = decltype(masked_c)::value;
        const int pos0 = tile * TOK + 4 * g;
        float x[2][8], mxs[2], rel[2];  // rel: the block's maximum relative to the running one (huge while there is none)
        bool raise = false;
#pragma unroll
        for (int gi = 0; gi < NG; ++gi) {
#pragma unroll
            for (int jj = 0; jj < 8; ++jj) x[gi][jj] = sc[gi][jj >> 2][jj & 3];  // raw dot products: the scale is folded into the exponent's multiply-add
            if (MASKED) {
                const int lim = row_pos[gi];
                const int low = sw > 0 ? max(0, lim + 1 - sw) : 0;
#pragma unroll
                for (int jj = 0; jj < 8; ++jj) {
                    const int pos = pos0 + 16 * (jj >> 2) + (jj & 3);
                    x[gi][jj] = (pos <= lim && pos >= low && kept[gi]) ? x[gi][jj] : -INFINITY;
                }
            }
            float mx = -INFINITY;
#pragma unroll
            for (int jj = 0; jj < 8; ++jj) mx = fmaxf(mx, x[gi][jj]);
            mxs[gi] = xor_max_g(mx) * scl;
            rel[gi] = mxs[gi] + neg_m[gi];  // (-inf for a row that sees nothing of this block)
            raise |= rel[gi] > 4.0f;
        }
        // The running maximum is only raised when a block exceeds it by more than 2^4: probabilities then stay below
        // 16 and the accumulators are rescaled a few times per row instead of once per block.
        if (__any(raise)) {
#pragma unroll
            for (int gi = 0; gi < NG; ++gi) {
                const float m_new = rel[gi] > 4.0f ? mxs[gi] : -neg_m[gi];
                const float d = -neg_m[gi] - m_new;  // 0 for a row that stays; -NO_MAX for one that held nothing (zeros)
                const float corr = __builtin_amdgcn_exp2f(d);
#pragma unroll
                for (int r = 0; r < RT; ++r) acc[gi][r] *= corr;
                l_part[gi] *= corr;
                lo_at[gi] += d;
                neg_m[gi] = -m_new;
                rel[gi] = mxs[gi] + neg_m[gi];
            }
        }
        bool need = false;
#pragma unroll
        for (int gi = 0; gi < NG; ++gi) {
#pragma unroll
            for (int jj = 0; jj < 8; ++jj) p[gi][jj] = __builtin_amdgcn_exp2f(fmaf(x[gi][jj], scl, neg_m[gi]));
#pragma unroll
            for (int jj = 0; jj < 4; ++jj) {
                uint32_t hi = pack2<DT>(p[gi][2 * jj], p[gi][2 * jj + 1]);
                if (DT == DT_BF16) asm("" : "+v"(hi));  // (its halves are taken from this word, not converted once more)
                pb[gi][jj] = hi;
                l_part[gi] = add_pair<DT>(hi, l_part[gi]);
                if constexpr (STASH) {
                    if (emit && gi == 0) {
                        // (head and token group of the lane from an opaque copy of the thread id: kept in registers of
                        // their own across the loop they would cost this variant a spill; pair by pair for the same
                        // reason)  LDS image: [tile of the item][head of the group][32 tokens], then [tile][head] maxima
                        int te_ = threadIdx.x;
                        asm volatile("" : "+v"(te_));
                        const int ne = te_ & 15, ge = (te_ >> 4) & 3;
                        if (ne < G) {
                            uint8_t* at = pkeep + ((j * G + ne) * TOK + 4 * ge + 16 * (jj >> 1) + 2 * (jj & 1)) * 2;
                            *reinterpret_cast<uint32_t*>(at) = pack2<DT_F16>(p[gi][2 * jj], p[gi][2 * jj + 1]);
                            if (jj == 0 && ge == 0)  // (a single-token row sees its item's first block, so it has a maximum)
                                *reinterpret_cast<float*>(pkeep + single_item_max_tiles(G) * G * TOK * 2 + (j * G + ne) * 4) = -neg_m[gi];
                        }
                    }
                }
            }
            need |= rel[gi] > lo_at[gi];
        }
        if constexpr (LO_ALWAYS) return true;
        if (!__any(need)) return false;
        // some row's largest probability is above the share of the denominator it was last compared with: look at the
        // denominators as they are now (this block included)
        need = false;
#pragma unroll
        for (int gi = 0; gi < NG; ++gi) {
            lo_at[gi] = __log2f(xor_sum_g(l_part[gi])) + LO_SHARE_LOG2;
            need |= rel[gi] > lo_at[gi];
        }
        return __any(need);
    };
    // what the rounding of the probabilities dropped, as operands of their own (and into the denominator)
    auto make_lo = [&](const u4v (&pb)[2], const float (&p)[2][8], u4v (&pl)[2]) __attribute__((always_inline)) {
#pragma unroll
        for (int gi = 0; gi < NG; ++gi)
#pragma unroll
            for (int jj = 0; jj < 4; ++jj) {
                const uint32_t hi = pb[gi][jj];  // (a bit cast straight from a vector element reads element 0)
                uint32_t lo;
                if (DT == DT_BF16) {
                    lo = pack2<DT>(p[gi][2 * jj] - __builtin_bit_cast(float, hi << 16),
                                   p[gi][2 * jj + 1] - __builtin_bit_cast(float, hi & 0xffff0000u));
                } else {
                    typedef _Float16 h2 __attribute__((ext_vector_type(2)));
                    const h2 h = __builtin_bit_cast(h2, hi);
                    lo = pack2<DT>(p[gi][2 * jj] - (float)h[0], p[gi][2 * jj + 1] - (float)h[1]);
                }
                pl[gi][jj] = lo;
                l_part[gi] = add_pair<DT>(lo, l_part[gi]);
            }
    };
    // O^T += V^T . P^T with one set of probability operands: sixteen (eight) independent accumulator tiles in a row
    auto pv_only = [&](const uint8_t* vb, const u4v (&pp)[2]) __attribute__((always_inline)) {
#pragma unroll
        for (int r = 0; r < RT; ++r) {
            const s8v vop = load_v(vb, r);
#pragma unroll
            for (int gi = 0; gi < NG; ++gi) acc[gi][r] = mma<DT>(vop, __builtin_bit_cast(s8v, pp[gi]), acc[gi][r]);
        }
    };

    // block number j start to end (QK, softmax, rescale, PV)
    auto body_whole = [&](auto masked_c, int j, const bool (&kept)[2], const uint8_t* kb, const uint8_t* vb)
                          __attribute__((always_inline)) {
        f4 sc[2][2];
        u4v pb[2], pl[2];
        if constexpr (U8) {
            float corr[2];
            qk_pv_at(true, kb, sc, false, vb, pb, pl);
            softmax(masked_c, sc, tile_at(j), j, pb, pl, corr, kept);
#pragma unroll
            for (int gi = 0; gi < NG; ++gi) {
                if (__any(corr[gi] != 1.0f)) {
#pragma unroll
                    for (int r = 0; r < RT; ++r) acc[gi][r] *= corr[gi];
                }
            }
            qk_pv_at(false, kb, sc, true, vb, pb, pl);
        } else {
            float p[2][8];
            qk_pv_at(true, kb, sc, false, vb, pb, pl);
            const bool lo = softmax16(masked_c, sc, tile_at(j), j, pb, p, kept);
            if constexpr (LO_ALWAYS) {  // both halves in one stream, each V operand read once
                make_lo(pb, p, pl);
                qk_pv_at(false, kb, sc, true, vb, pb, pl);
            } else {
                if (lo) make_lo(pb, p, pl);
                pv_only(vb, pb);
                if (lo) pv_only(vb, pl);
            }
        }
    };
    auto whole_at = [&](int j, const uint8_t* kb, const uint8_t* vb) __attribute__((always_inline)) {
        const int tile = tile_at(j);
        bool kept[2] = {true, true};
        if constexpr (XATT) {
            const int k = (tile >> xt_shift) - kb_lo;
#pragma unroll
            for (int gi = 0; gi < NG; ++gi) {
                kept[gi] = (row_keep[4 * (16 * NG * wv + 16 * gi + n) + (k >> 5)] >> (k & 31)) & 1u;
            }
        }
        if (XATT || tile * TOK < free_lo || tile * TOK + TOK - 1 > free_hi)  // wave-uniform
            body_whole(std::true_type{}, j, kept, kb, vb);
        else
            body_whole(std::false_type{}, j, kept, kb, vb);
    };
    auto whole = [&](int j) __attribute__((always_inline)) {
        whole_at(j, smem + kslot(j) * TILEK, smem + OFF_V + vslot(j) * TILEV);
    };

    if constexpr (DMA) {
        // Block number j lives in K slot and V slot j % 4.  A wave moves rows 8 wv .. 8 wv + 7 of a block: lane l of
        // its two instructions per tensor takes row 8 wv + 4 i + l / 16, LDS piece position l % 16, i.e. the row's
        // piece (l % 16) ^ (row & 15) of K, (l % 16) ^ 2 (row & 7) of V.  Every step issues the same four copies per
        // wave (indices clamped), so that "at most eight outstanding" always means: everything but the two youngest
        // blocks has landed.
        const int wvs = __builtin_amdgcn_readfirstlane(wv);
        const int my_row = 8 * wvs + (lane >> 4);         // + 4 for the second instruction
        // per-lane byte offsets within a block (32 bits, added to a wave-uniform block address)
        const uint32_t off_k0 = my_row * ROWB + (((lane & 15) ^ (my_row & 15)) << 4);
        const uint32_t off_k1 = (my_row + 4) * ROWB + (((lane & 15) ^ ((my_row + 4) & 15)) << 4);
        const uint32_t off_v0 = my_row * ROWB + (((lane & 15) ^ ((my_row & 7) << 1)) << 4);
        const uint32_t off_v1 = (my_row + 4) * ROWB + (((lane & 15) ^ (((my_row + 4) & 7) << 1)) << 4);
        const bool upper_half = wvs >= (NT / 64) / 2;  // this wave moves rows 16 - 31
        // The table entry of a copy's block is read one step before the copy goes out, and nothing is computed from it
        // until then: a scalar load that is waited for right behind its issue stalls the wave at every step.
        auto table_index = [&](int tile) __attribute__((always_inline)) {
            return bs16 ? min(2 * tile + (upper_half ? 1 : 0), last_block16) : tile >> sub_shift;
        };
        int id_next = table[table_index(tile_at(0))];
        auto copy_in = [&](int j, uint8_t* kslot_base, uint8_t* vslot_base) __attribute__((always_inline)) {
            const int tile = tile_at(j);
            // (what tile_base gives for this wave's half of the tile, from the entry read a step ago)
            const long blk = bs16 ? ((long)id_next * Hkv + hkv) * (16 * CROWB) - (upper_half ? 16 * CROWB : 0)
                                  : ((long)id_next * Hkv + hkv) * ((long)a.sh.bs * CROWB) + (long)(tile & sub_mask) * (TOK * CROWB);
            id_next = table[table_index(tile_at(j + 1))];
            const uint8_t* kg = a.key_cache + blk;
            const uint8_t* vg = a.value_cache + blk;
            uint8_t* kd = kslot_base + wvs * 2048;
            uint8_t* vd = vslot_base + wvs * 2048;
            dma16(kg + off_k0, kd);
            dma16(kg + off_k1, kd + 1024);
            dma16(vg + off_v0, vd);
            dma16(vg + off_v1, vd + 1024);
        };
        // The wait in front of a step's barrier names how many of the wave's vector-memory operations may still be
        // outstanding: the copies of the two youngest blocks.  It is only right while a step issues exactly this many
        // copies per wave and nothing else that counts (the table reads above are scalar loads; the build fails on
        // spills, whose scratch traffic would count).
        constexpr int COPIES_PER_STEP = 4;
        static_assert(COPIES_PER_STEP == 2 * (TOK * ROWB / 1024) / (NT / 64), "copy_in issues one 1024-byte copy per 8 rows of K and of V for each wave");
        copy_in(0, dk0, dv0);
        copy_in(1, dk1, dv1);
        copy_in(2, dk2, dv2);
        // the query loads (issued above, tracked by the compiler) are waited for here, not inside the loop
#pragma unroll
        for (int gi = 0; gi < NG; ++gi)
#pragma unroll
            for (int s = 0; s < KS; ++s) asm volatile("" ::"v"(qreg[gi][s]));
        // step j: block j sits in slot j % 4 (kc, vc); the slot of block j - 1 (kn, vn) takes block j + 3
#define PA_DMA_STEP(kc, vc, kn, vn)                                                                      \
        {                                                                                                \
            if (j >= cnt) break;                                                                         \
            wait_vmem<2 * COPIES_PER_STEP>();  /* this wave's part of block j has landed (blocks j + 1, j + 2 may be on their way) */ \
            lds_barrier();   /* so has everyone else's, and block j - 1 is done with */                  \
            copy_in(j + 3, kn, vn);                                                                      \
            const int tile = tile_at(j);                                                                 \
            if (tile * TOK + TOK > kv_len) { /* (uniform) the sequence's last block: clear the V rows beyond its tokens */ \
                for (int c = tid; c < (TOK - (kv_len - tile * TOK)) * CPR; c += NT)                       \
                    *reinterpret_cast<u4v*>(vc + (kv_len - tile * TOK) * LROWV + c * 16) = u4v{0u, 0u, 0u, 0u}; \
                lds_barrier();                                                                           \
            }                                                                                            \
            if (active) whole_at(j, kc, vc);                                                             \
            ++j;                                                                                         \
        }
        for (int j = 0;;) {
            PA_DMA_STEP(dk0, dv0, dk3, dv3)
            PA_DMA_STEP(dk1, dv1, dk0, dv0)
            PA_DMA_STEP(dk2, dv2, dk1, dv1)
            PA_DMA_STEP(dk3, dv3, dk2, dv2)
        }
#undef PA_DMA_STEP
        wait_vmem<0>();  // the clamped copies of the last three steps still target this workgroup's LDS
    } else if constexpr (HALF) {
        // Two register sets: block j + 2 goes from its set to LDS at the start of step j and the set takes block j + 4
        // right behind it (the same two steps between a fetch and its use as with three sets, 16 registers fewer).
        fetch(set[0], 0);
        fetch(set[1], 1);
#pragma unroll
        for (int gi = 0; gi < NG; ++gi)
#pragma unroll
            for (int s = 0; s < KS; ++s) asm volatile("" ::"v"(qreg[gi][s]));
        stash(set[0], 0);
        fetch(set[0], 2);
        stash(set[1], 1);
        fetch(set[1], 3);
        __syncthreads();
        if (active && cnt > 0) whole(0);
        __syncthreads();
        for (int j = 0; j < cnt; j += 2) {
            stash(set[0], j + 2);
            fetch(set[0], j + 4);
            if (active && j + 1 < cnt) whole(j + 1);
            __syncthreads();
            if (j + 1 >= cnt) break;
            stash(set[1], j + 3);
            fetch(set[1], j + 5);
            if (active && j + 2 < cnt) whole(j + 2);
            __syncthreads();
        }
    } else {
        fetch(set[0], 0);
        fetch(set[1], 1);
        fetch(set[2], 2);
        // step 0 multiplies V slot 3 by zero probabilities: make sure it holds numbers
#pragma unroll
        for (int uu = 0; uu < UPT; ++uu)
            if (unit_loads(uu)) *reinterpret_cast<u4v*>(smem + 3 * TILEV + unit_lds_v(uu)) = u4v{0u, 0u, 0u, 0u};
        // the query loads (issued above, tracked by the compiler) are waited for here, not inside the loop
    #pragma unroll
        for (int gi = 0; gi < NG; ++gi)
    #pragma unroll
            for (int s = 0; s < KS; ++s) asm volatile("" ::"v"(qreg[gi][s]));
        stash(set[0], 0);
        fetch(set[0], 3);
        stash(set[1], 1);
        __syncthreads();
        if (active && cnt > 0) whole(0);  // (a block-sparse item may have nothing left to do)
        __syncthreads();  // step 0 overwrites K slot 0, which the lines above read
        // step j: set (j+1)%3 was written to LDS in step j-1 and takes block t+4; set (j+2)%3 holds block t+2; the
        // step works on block t+1 (whose K and V are both in LDS by then); block tb was done above.
    #define PA_STEP(K)                                                                       \
        {                                                                                    \
            const int j = i + K;                                                             \
            if (j >= cnt) break;                                                             \
            fetch(set[(K + 1) % 3], j + 4);                                                  \
            if (active && j + 1 < cnt) whole(j + 1);                                         \
            stash(set[(K + 2) % 3], j + 2);                                                  \
            __syncthreads();                                                                 \
        }
        for (int i = 0;; i += 3) {
            PA_STEP(0)
            PA_STEP(1)
            PA_STEP(2)
        }
    #undef PA_STEP
    }

    // ---- write the rows ------------------------------------------------------------------------------
    if constexpr (!U8) {
#pragma unroll
        for (int gi = 0; gi < NG; ++gi) m_run[gi] = neg_m[gi] == NO_MAX ? -INFINITY : -neg_m[gi];
    }
    const bool final_out = item.nsplit == 1;
    // the lane's group number again, from an opaque copy of the thread id: nothing inside the loop reads it, and kept
    // alive across the loop it costs the variants that sit at their register limit a spill
    int ge = threadIdx.x;
    asm volatile("" : "+v"(ge));
    if constexpr (STASH) {  // ... and the row's id, for the same reason (one row group per wave)
        const int rho = min(16 * (ge >> 6) + (ge & 15), R - 1);
        row_id[0] = (t0 + q0 + rho / G) * Hq + hkv * G + rho % G;
    }
    ge = (ge >> 4) & 3;
#pragma unroll
    for (int gi = 0; gi < NG; ++gi) {
        const float l = xor_sum_g(l_part[gi]);
        if (U8) {  // code units back to values, minus the zero-point term
            const float z = xor_sum_g(zsum[gi]);
#pragma unroll
            for (int r = 0; r < RT; ++r) acc[gi][r] = acc[gi][r] * CODE_UNIT - z;
        }
        if (row_pos[gi] < 0) continue;
        // register i of tile r on lane (n, g) holds channel 16 r + 4 g + i of row n
        if (final_out) {
            const float inv = l > 0.0f ? 1.0f / l : 0.0f;
            uint16_t* o = a.out + (long)row_id[gi] * D;
#pragma unroll
            for (int r = 0; r < RT; ++r)
                *reinterpret_cast<uint2*>(o + 16 * r + 4 * ge) =
                    make_uint2(pack2<QDT>(acc[gi][r][0] * inv, acc[gi][r][1] * inv),
                               pack2<QDT>(acc[gi][r][2] * inv, acc[gi][r][3] * inv));
            if (ge == 0) {  // natural-log maximum and denominator for the score kernels
                a.final_ml[2 * (long)row_id[gi]] = m_run[gi] * LN2;
                a.final_ml[2 * (long)row_id[gi] + 1] = l;
            }
        } else {
            const long slot = (long)row_id[gi] * a.max_split + item.split;
            float* o = a.part_acc + slot * D;
#pragma unroll
            for (int r = 0; r < RT; ++r) *reinterpret_cast<f4*>(o + 16 * r + 4 * ge) = acc[gi][r];
            if (ge == 0) {
                a.part_ml[2 * slot] = m_run[gi];
                a.part_ml[2 * slot + 1] = l;
            }
        }
    }
    if constexpr (STASH) {
        if (emit) {  // (uniform) behind the rows, with their registers free: the item's probabilities and maxima: LDS -> [tile][Hq][32] / [tile][Hq]
            __syncthreads();
            const long tile0 = tile_max_offset(st.score_offsets[b], b) + tb;
            int te_ = threadIdx.x;
            asm volatile("" : "+v"(te_));
            for (int i = te_; i < cnt * G * (TOK / 8); i += NT) {  // 16-byte pieces
                const int piece = i % (TOK / 8), h = (i / (TOK / 8)) % G, jt = i / (TOK / 8) / G;
                *reinterpret_cast<u4v*>(a.p_out + ((tile0 + jt) * Hq + hkv * G + h) * TOK + piece * 8) =
                    *reinterpret_cast<const u4v*>(pkeep + ((jt * G + h) * TOK + piece * 8) * 2);
            }
            for (int i = te_; i < cnt * G; i += NT)
                a.tile_max[(tile0 + i / G) * Hq + hkv * G + i % G] =
                    *reinterpret_cast<const float*>(pkeep + single_item_max_tiles(G) * G * TOK * 2 + i * 4);
        }
    }
}

// Rows whose context was cut into several ranges: fold the partials (maxima in the log2 domain).
template <int D, int DT>
__global__ __launch_bounds__(256) void pa_prefill16_merge_kernel(MergeRows m) {
    merge_rows<D, DT>(m, blockIdx.x);
}

}  // namespace

template <int D, int DT, int QDT, bool U8>
static hipError_t launch_prefill16_typed(hipStream_t s, const PrefillArgs& a, hipEvent_t ev0, hipEvent_t ev1,
                                         bool merge_later) {
    if (ev0) (void)hipEventRecord(ev0, s);
    if constexpr (U8 && D != 96 && D != 256) {
        if (a.n_wide > 0) {  // u8 caches: the items with more than 16 query rows (up to 128) come first in the list
            PrefillArgs w = a;
            w.n_items = a.n_wide;
            hipLaunchKernelGGL((pa_prefill16_kernel<D, DT, QDT, U8, 2, false, false, true>), dim3((unsigned)w.n_items * a.sh.Hkv), dim3(256), 0, s, w);
        }
    } else if (a.n_wide > 0) {
        return hipErrorInvalidValue;  // (16-bit caches list no such group)
    }
    const int n_narrow = a.n_items - a.n_sparse - a.n_wide - (a.skip_single ? a.n_single : 0);
    if (n_narrow > 0) {  // the rest of the dense ones, listed behind them
        PrefillArgs nrw = a;
        nrw.items = a.items + a.n_wide;
        nrw.n_items = n_narrow;
        // 16-bit caches, head size 128, chunks only: blocks straight into LDS, two row groups per wave.  (Items of
        // single-token sequences hold a handful of rows: next to them the one-group variant, with more waves moving
        // blocks and half the arithmetic on empty rows, is the faster one -- 0.25 against 0.31 ms on the mixed workload.)
        bool straight = false;
        if constexpr (!U8 && D == 128) straight = a.n_single == 0 || a.skip_single;
        if constexpr (!U8 && D == 128) {
            if (straight)
                hipLaunchKernelGGL((pa_prefill16_kernel<D, DT, QDT, U8, 2, false, true>), dim3((unsigned)nrw.n_items * a.sh.Hkv), dim3(256), 0, s, nrw);
        }
        if (!straight)
            hipLaunchKernelGGL((pa_prefill16_kernel<D, DT, QDT, U8, 1, false, false>), dim3((unsigned)nrw.n_items * a.sh.Hkv), dim3(512), 0, s, nrw);
    }
    if (a.n_sparse > 0) {  // the items of block-sparse sequences come last
        PrefillArgs sp = a;
        sp.items = a.items + (a.n_items - a.n_sparse);
        sp.n_items = a.n_sparse;
        // 128 query rows per workgroup whatever the cache: the fewer tokens share a work item, the fewer KV blocks
        // it has to walk for rows that did not keep them
        hipLaunchKernelGGL((pa_prefill16_kernel<D, DT, QDT, U8, 1, true, false>), dim3((unsigned)sp.n_items * a.sh.Hkv), dim3(512), 0, s, sp);
    }
    if (ev1) (void)hipEventRecord(ev1, s);
    if (a.n_merge > 0 && !merge_later) {
        const MergeRows m = merge_rows_of(a);
        hipLaunchKernelGGL((pa_prefill16_merge_kernel<D, QDT>), dim3((unsigned)m.n_wg), dim3(256), 0, s, m);
    }
    return hipGetLastError();
}

template <int D>
static hipError_t launch_prefill16_d(hipStream_t s, const PrefillArgs& a, int q_dtype, int kv_dtype, hipEvent_t ev0,
                                     hipEvent_t ev1, bool merge_later) {
    if (kv_dtype == DT_U8)
        return q_dtype == DT_F16 ? launch_prefill16_typed<D, DT_F16, DT_F16, true>(s, a, ev0, ev1, merge_later)
                                 : launch_prefill16_typed<D, DT_F16, DT_BF16, true>(s, a, ev0, ev1, merge_later);
    if (kv_dtype != q_dtype) return hipErrorInvalidValue;
    return q_dtype == DT_F16 ? launch_prefill16_typed<D, DT_F16, DT_F16, false>(s, a, ev0, ev1, merge_later)
                             : launch_prefill16_typed<D, DT_BF16, DT_BF16, false>(s, a, ev0, ev1, merge_later);
}

hipError_t launch_prefill16(hipStream_t s, const PrefillArgs& a, int q_dtype, int kv_dtype, hipEvent_t ev0,
                            hipEvent_t ev1, bool merge_later) {
    if (a.n_items == 0) return hipSuccess;
    if (a.sh.D == 128) return launch_prefill16_d<128>(s, a, q_dtype, kv_dtype, ev0, ev1, merge_later);
    if (a.sh.D == 64) return launch_prefill16_d<64>(s, a, q_dtype, kv_dtype, ev0, ev1, merge_later);
    if (a.sh.D == 96) return launch_prefill16_d<96>(s, a, q_dtype, kv_dtype, ev0, ev1, merge_later);
    if (a.sh.D == 256) return launch_prefill16_d<256>(s, a, q_dtype, kv_dtype, ev0, ev1, merge_later);
    return hipErrorInvalidValue;
}

}  // namespace pa
