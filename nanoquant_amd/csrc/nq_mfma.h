// Pieces shared by the prefill kernels: the MFMA wrappers and the constants of the packed weight tiles.
#pragma once
#include "nq_common.h"

namespace nq {

typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));

constexpr int kTileK = 256;  // k extent of one packed weight tile (and the granularity of k-splits)

// LDS row pitch in 16-bit elements for a slab of KS k-values: 16 bytes of padding make the 128-bit
// fragment reads of 32 consecutive rows conflict-free.
template <int KS>
constexpr int slab_pitch() { return KS + 8; }

template <int DT>
struct Mfma;
template <>
struct Mfma<0> {
    static __device__ __forceinline__ float16_t run(uint4 a, uint4 b, float16_t c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(half8_t, a), __builtin_bit_cast(half8_t, b), c, 0, 0, 0);
    }
};
template <>
struct Mfma<1> {
    static __device__ __forceinline__ float16_t run(uint4 a, uint4 b, float16_t c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf168_t, a), __builtin_bit_cast(bf168_t, b), c, 0, 0, 0);
    }
};

__device__ __forceinline__ uint32_t comp4(const uint4& v, int i) {
    return i == 0 ? v.x : i == 1 ? v.y : i == 2 ? v.z : v.w;
}

// Raw buffer view (gfx9 resource words) of `bytes` bytes at p: loads past the end return zeros and stores past
// the end are dropped, so a lane with nothing to do is pointed past the end instead of being branched around.
__device__ __forceinline__ __amdgpu_buffer_rsrc_t gemm_buffer(const void* p, uint32_t bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), 0, (int)bytes, 0x00020000);
}
constexpr int kGemmCacheDefault = 0;
constexpr int kGemmCacheAgent = 16;   // sc1: coherent at device scope (not served from this XCD's L2)

}  // namespace nq
