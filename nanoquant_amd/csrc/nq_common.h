// Shared device helpers for the gfx950 binary low-rank kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>

namespace nq {

// Host side: "done once on this device" for settings that HIP keeps per device (function attributes) and for values
// queried per device.  One bit per device ordinal; devices beyond 63 simply repeat the (idempotent) work.  Safe for
// concurrent first calls: two threads may both do the work, none skips it.
struct PerDeviceFlag {
    std::atomic<unsigned long long> bits{0};
    bool test(int dev) const { return dev >= 0 && dev < 64 && ((bits.load(std::memory_order_acquire) >> dev) & 1ull); }
    void set(int dev) {
        if (dev >= 0 && dev < 64) bits.fetch_or(1ull << dev, std::memory_order_release);
    }
};
inline int current_device() {
    int dev = -1;
    return hipGetDevice(&dev) == hipSuccess ? dev : -1;
}

typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef __bf16 bf162_t __attribute__((ext_vector_type(2)));
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef __bf16 bf168_t __attribute__((ext_vector_type(8)));
typedef float float4_t __attribute__((ext_vector_type(4)));
typedef float float16_t __attribute__((ext_vector_type(16)));

constexpr int kWave = 64;
constexpr uint32_t kSignPair = 0x80008000u;

// Element traits.  DT = 0: IEEE fp16, DT = 1: bfloat16.  Values travel as raw 16-bit patterns so
// that the sign can be flipped with integer logic, as the packed "half2" word order intends.
template <int DT>
struct Elem;

template <>
struct Elem<0> {
    static constexpr uint32_t kOnePair = 0x3C003C00u;  // (1.0h, 1.0h)
    static constexpr uint32_t kOne = 0x3C00u;
    static __device__ __forceinline__ float dot2(uint32_t a, uint32_t b, float c) {
        return __builtin_amdgcn_fdot2(__builtin_bit_cast(half2_t, a), __builtin_bit_cast(half2_t, b), c, false);
    }
    static __device__ __forceinline__ float to_float(uint16_t v) {
        return (float)__builtin_bit_cast(_Float16, v);
    }
    static __device__ __forceinline__ uint16_t from_float(float f) {
        return __builtin_bit_cast(uint16_t, (_Float16)f);
    }
    // Final store of the decode path: clamp as the reference does (kernel/cuda/cuda_utils.cuh:83-86).
    static __device__ __forceinline__ uint16_t from_float_clamped(float f) {
        return from_float(fminf(fmaxf(f, -64504.0f), 64504.0f));
    }
    // Final store of the prefill path: saturate to the largest finite fp16.
    static __device__ __forceinline__ uint16_t from_float_sat(float f) {
        return from_float(fminf(fmaxf(f, -65504.0f), 65504.0f));
    }
};

template <>
struct Elem<1> {
    static constexpr uint32_t kOnePair = 0x3F803F80u;  // (1.0bf, 1.0bf)
    static constexpr uint32_t kOne = 0x3F80u;
    static __device__ __forceinline__ float dot2(uint32_t a, uint32_t b, float c) {
        return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf162_t, a), __builtin_bit_cast(bf162_t, b), c,
                                               false);
    }
    static __device__ __forceinline__ float to_float(uint16_t v) {
        return __builtin_bit_cast(float, (uint32_t)v << 16);
    }
    static __device__ __forceinline__ uint16_t from_float(float f) {
        return __builtin_bit_cast(uint16_t, (__bf16)f);
    }
    static __device__ __forceinline__ uint16_t from_float_clamped(float f) {
        return from_float(fminf(fmaxf(f, -3.3895313892515355e+38f), 3.3895313892515355e+38f));
    }
    static __device__ __forceinline__ uint16_t from_float_sat(float f) { return from_float_clamped(f); }
};

// Workgroup barrier that orders LDS traffic only.  __syncthreads() also waits for every outstanding
// global load of the wavefront (vmcnt counts loads and stores alike), which would serialise a prefetch
// that is deliberately kept in flight across the barrier.
__device__ __forceinline__ void lds_barrier() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

// ---- cross-lane sums on a 64-wide wavefront -------------------------------------------------
// DPP control words (gfx9 encoding): quad_perm = 4 x 2-bit selects; 0x140 row_mirror;
// 0x141 row_half_mirror.
template <int CTRL>
__device__ __forceinline__ float dpp_add(float v) {
    int moved = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, false);
    return v + __builtin_bit_cast(float, moved);
}

// Sum over aligned groups of `group` consecutive lanes (group = 1,2,4,...,64; wave-uniform).  Every
// lane of a group ends up with the group's total.  Steps inside a 16-lane row are DPP moves; the
// two cross-row steps go through the LDS crossbar (ds_bpermute), no LDS memory involved.
__device__ __forceinline__ float group_sum(float v, int group) {
    if (group >= 2) v = dpp_add<0xB1>(v);   // quad_perm [1,0,3,2]
    if (group >= 4) v = dpp_add<0x4E>(v);   // quad_perm [2,3,0,1]
    if (group >= 8) v = dpp_add<0x141>(v);  // row_half_mirror: lane i <-> 7-i within 8
    if (group >= 16) v = dpp_add<0x140>(v); // row_mirror: lane i <-> 15-i within 16
    if (group >= 32) v += __shfl_xor(v, 16, kWave);
    if (group >= 64) v += __shfl_xor(v, 32, kWave);
    return v;
}

// Sum over aligned groups of 16, 32 or 64 lanes with DPP moves only (no LDS crossbar).  The total is
// valid in the LAST 16 lanes of every group; the other lanes hold partial sums.  0x142 = row_bcast15
// (lane 15 of a row to the next row), 0x143 = row_bcast31 (lane 31 to rows 2 and 3).
__device__ __forceinline__ float group_sum_tail(float v, int group) {
    v = dpp_add<0xB1>(v);
    v = dpp_add<0x4E>(v);
    v = dpp_add<0x141>(v);
    v = dpp_add<0x140>(v);       // every lane: the total of its 16-lane row
    if (group >= 32) {
        const int moved = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x142, 0xA, 0xF, false);
        v += __builtin_bit_cast(float, moved);
    }
    if (group >= 64) {
        const int moved = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x143, 0xC, 0xF, false);
        v += __builtin_bit_cast(float, moved);
    }
    return v;
}

}  // namespace nq
