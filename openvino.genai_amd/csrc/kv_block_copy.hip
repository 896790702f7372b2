// Copy-on-write of KV blocks: every (source, destination) pair of a call, in every layer's K and V tensor, in one
// launch.  HBM-bound byte work: each block byte is read once and written once, 16 bytes per lane, fully coalesced.
#include "pa_device.h"

namespace pa {
namespace {

typedef uint32_t u4v __attribute__((ext_vector_type(4)));
constexpr int COPY_UNROLL = 4;  // 16-byte pieces per thread

// grid = (pieces of a block, pair, tensor); `bases` holds the tensors' base addresses (K and V of every layer),
// `tensor_block_bytes` the size of a block in each of them (tensors may differ in head size and element type)
__global__ __launch_bounds__(256) void kv_copy_blocks_kernel(uint8_t* const* __restrict__ bases,
                                                             const uint64_t* __restrict__ tensor_block_bytes,
                                                             const int2* __restrict__ pairs) {
    const int2 p = pairs[blockIdx.y];
    uint8_t* base = bases[blockIdx.z];
    const long block_bytes = (long)tensor_block_bytes[blockIdx.z];
    const u4v* src = reinterpret_cast<const u4v*>(base + (long)p.x * block_bytes);
    u4v* dst = reinterpret_cast<u4v*>(base + (long)p.y * block_bytes);
    const long n16 = block_bytes / 16;
    const long i0 = ((long)blockIdx.x * COPY_UNROLL) * 256 + threadIdx.x;
    u4v v[COPY_UNROLL];
#pragma unroll
    for (int u = 0; u < COPY_UNROLL; ++u)
        if (i0 + u * 256 < n16) v[u] = src[i0 + u * 256];
#pragma unroll
    for (int u = 0; u < COPY_UNROLL; ++u)
        if (i0 + u * 256 < n16) dst[i0 + u * 256] = v[u];
}

}  // namespace

// Every tensor's block size is a multiple of 16 (the caller checks); `max_block_bytes` is the largest of them.
hipError_t launch_copy_blocks(hipStream_t s, void* const* bases, const uint64_t* tensor_block_bytes, int n_tensors,
                              const int32_t* pairs, int count, size_t max_block_bytes) {
    if (count <= 0 || n_tensors <= 0) return hipSuccess;
    const long n16 = (long)(max_block_bytes / 16);
    const unsigned gx = (unsigned)((n16 + 256 * COPY_UNROLL - 1) / (256 * COPY_UNROLL));
    for (int c0 = 0; c0 < count; c0 += 65535) {  // grid y
        const int c = count - c0 < 65535 ? count - c0 : 65535;
        hipLaunchKernelGGL(kv_copy_blocks_kernel, dim3(gx, (unsigned)c, (unsigned)n_tensors), dim3(256), 0, s,
                           reinterpret_cast<uint8_t* const*>(bases), tensor_block_bytes,
                           reinterpret_cast<const int2*>(pairs) + c0);
    }
    return hipGetLastError();
}

}  // namespace pa
