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

// Row-major words (either order) -> the 32-row x 256-k tiles of the prefill kernels, no dense matrix in between.
// Tile (rt, kt) is 64 lanes x 4 words; lane l owns row 32 rt + (l & 31), its word q holds, at in-word element
// j = 8 t + e (t = 0..3, e = 0..7; "half2" bit position), the column k = 256 kt + 64 q + 16 t + 8 (l >> 5) + e.
// So an output word draws 16 elements from each of the source words 8 kt + 2 q and 8 kt + 2 q + 1 of its row.
// Rows beyond `rows` and words beyond `words` read as zero words (= +1 signs), which is the rank padding of the
// two-stage packer.  One thread per output word.
__global__ __launch_bounds__(256) void words_to_tiles_kernel(const uint32_t* __restrict__ src, uint32_t* __restrict__ dst,
                                                             int rows, int words, int ktiles, int src_order, size_t nout) {
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < nout; i += stride) {
        const int q = (int)(i & 3), l = (int)((i >> 2) & 63);
        const size_t tile = i >> 8;
        const int kt = (int)(tile % (size_t)ktiles), rt = (int)(tile / (size_t)ktiles);
        const int row = 32 * rt + (l & 31), half = l >> 5;
        const int w0 = 8 * kt + 2 * q;
        uint32_t s[2] = {0u, 0u};
        if (row < rows) {
            if (w0 < words) s[0] = src[(size_t)row * words + w0];
            if (w0 + 1 < words) s[1] = src[(size_t)row * words + w0 + 1];
        }
        uint32_t o = 0;
#pragma unroll
        for (int j = 0; j < 32; ++j) {
            const int t = j >> 3, e = j & 7;
            const int elem = 16 * (t & 1) + 8 * half + e;          // element of source word t >> 1
            o |= ((s[t >> 1] >> word_bit(elem, src_order)) & 1u) << word_bit(j, 1);
        }
        dst[i] = o;
    }
}

hipError_t words_to_tiles(const uint32_t* src, uint32_t* dst, int rows, int words, int rows_padded, int k_padded,
                          int src_order, hipStream_t stream) {
    const size_t nout = (size_t)rows_padded * k_padded / 32;
    if (nout == 0) return hipSuccess;
    size_t blocks = (nout + 255) / 256;
    if (blocks > 256 * 16) blocks = 256 * 16;
    hipLaunchKernelGGL(words_to_tiles_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, src, dst, rows, words,
                       k_padded / 256, src_order, nout);
    return hipGetLastError();
}

// Tile order of the run-list kernel: 16-byte units (4 words) indexed [row / 32][unit / 4][(row / 16) & 1][unit & 3]
// [row & 15], rows padded to a multiple of 32 and units to a multiple of 4 with zero words.  The 64 units that
// one wavefront fetches for an MFMA operand (16 rows x 4 units) are 1 KiB contiguous, the two row groups of a
// 32-row pair adjacent.  One thread per destination (tile: tiled, else row-major) unit.
__host__ __device__ __forceinline__ size_t tiled_unit_index(int row, int unit, int groups) {
    return (((((size_t)(row >> 5) * groups + (unit >> 2)) * 2 + ((row >> 4) & 1)) * 4 + (unit & 3)) * 16) + (row & 15);
}

size_t tiled_word_count(int rows, int words) {
    const size_t groups = ((size_t)words + 15) / 16;
    return (((size_t)rows + 31) / 32) * groups * 128 * 4;
}

__global__ __launch_bounds__(256) void tile_kernel(const uint32_t* src, uint32_t* dst, int rows, int words, int groups,
                                                   int inverse, size_t nunits) {
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < nunits; i += stride) {
        if (!inverse) {
            // i = tiled unit index -> (row, unit)
            const int r16 = (int)(i & 15), g = (int)((i >> 4) & 3), half = (int)((i >> 6) & 1);
            const size_t t = i >> 7;
            const int ub = (int)(t % (size_t)groups), rp = (int)(t / (size_t)groups);
            const int row = 32 * rp + 16 * half + r16, unit = 4 * ub + g;
            uint32_t w[4];
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const int c = 4 * unit + k;
                w[k] = (row < rows && c < words) ? src[(size_t)row * words + c] : 0u;
            }
            ((uint4*)dst)[i] = make_uint4(w[0], w[1], w[2], w[3]);
        } else {
            // i = row-major unit index over [rows][ceil(words / 4)]
            const int upr = (words + 3) / 4;
            const int row = (int)(i / (size_t)upr), unit = (int)(i % (size_t)upr);
            const uint4 v = ((const uint4*)src)[tiled_unit_index(row, unit, groups)];
            const uint32_t w[4] = {v.x, v.y, v.z, v.w};
            for (int k = 0; k < 4; ++k)
                if (4 * unit + k < words) dst[(size_t)row * words + 4 * unit + k] = w[k];
        }
    }
}

hipError_t tile_words(const uint32_t* src, uint32_t* dst, int rows, int words, int inverse, hipStream_t stream) {
    if (rows <= 0 || words <= 0) return hipSuccess;
    const int groups = (words + 15) / 16;
    const size_t nunits = inverse ? (size_t)rows * ((words + 3) / 4) : tiled_word_count(rows, words) / 4;
    size_t blocks = (nunits + 255) / 256;
    if (blocks > 256 * 16) blocks = 256 * 16;
    hipLaunchKernelGGL(tile_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, src, dst, rows, words, groups, inverse, nunits);
    return hipGetLastError();
}

}  // namespace nq
