// Small memory-bound helpers: a plain copy kernel of known traffic and the per-word bit permutation
// between the two row-major word orders.
#include "nq_common.h"
#include "nq_kernels.h"

namespace nq {

__global__ __launch_bounds__(256) void copy_kernel(uint4* __restrict__ dst, const uint4* __restrict__ src, size_t n16) {
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n16; i += stride) dst[i] = src[i];
}

hipError_t stream_copy(void* dst, const void* src, size_t bytes, hipStream_t stream) {
    const size_t n16 = bytes / 16;
    if (n16 == 0) return hipSuccess;
    size_t blocks = (n16 + 255) / 256;
    if (blocks > 256 * 16) blocks = 256 * 16;
    hipLaunchKernelGGL(copy_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, (uint4*)dst, (const uint4*)src, n16);
    return hipGetLastError();
}

// Bit index of element k (0..31) of a 32-group.  order 0: lsb_first (bit k); order 1: half2
// (even elements fill bits 15..0 downwards, odd elements bits 31..16 downwards).
__host__ __device__ __forceinline__ int word_bit(int k, int order) {
    return order == 0 ? k : 15 - (k >> 1) + 16 * (k & 1);
}

__global__ __launch_bounds__(256) void repack_kernel(const uint32_t* src, uint32_t* dst, size_t n, int so, int d_o) {
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
        const uint32_t w = src[i];
        uint32_t o = 0;
#pragma unroll
        for (int k = 0; k < 32; ++k) o |= ((w >> word_bit(k, so)) & 1u) << word_bit(k, d_o);
        dst[i] = o;
    }
}

hipError_t repack_words(const uint32_t* src, uint32_t* dst, size_t nwords, int src_order, int dst_order,
                        hipStream_t stream) {
    if (nwords == 0) return hipSuccess;
    size_t blocks = (nwords + 255) / 256;
    if (blocks > 256 * 16) blocks = 256 * 16;
    hipLaunchKernelGGL(repack_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, src, dst, nwords, src_order, dst_order);
    return hipGetLastError();
}

}  // namespace nq
