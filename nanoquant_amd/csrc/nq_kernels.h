// Internal launch interface between the C-ABI layer (nq_api.hip) and the kernel files.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace nq {

// nq_gemv.hip: one matmul-free stage.  dtype 0 = fp16, 1 = bf16.  first: input is 16-bit activations
// scaled by s_col; otherwise input is the fp32 intermediate.  Output is fp32 when out_f32, else the
// activation type (clamped); `addend` (fp32, same shape as out) is added before the store.
hipError_t gemv_stage(int dtype, bool first, const uint32_t* bits, const void* in, const void* s_col,
                      const void* s_row, const float* addend, void* out, bool out_f32, int batch, int rows,
                      int words, int K, int in_stride, int out_stride, hipStream_t stream);

// nq_gemm.hip: C[T,R] = s_out * ((x * s_in) . sgn(W)^T) with W in the 32x256 tile layout.
// scratch: fp32 [T,R] when gemm_scratch_bytes(T,K,R) > 0.
size_t gemm_scratch_bytes(int T, int K, int R);
hipError_t gemm_onebit(int dtype, const void* x, const uint32_t* tiles, const void* s_in, const void* s_out,
                       void* y, float* scratch, int T, int K, int R, hipStream_t stream);

// nq_util.hip
hipError_t stream_copy(void* dst, const void* src, size_t bytes, hipStream_t stream);
hipError_t repack_words(const uint32_t* src, uint32_t* dst, size_t nwords, int src_order, int dst_order,
                        hipStream_t stream);

}  // namespace nq
