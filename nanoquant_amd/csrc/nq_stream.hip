// Decode path, run-list form: ONE persistent launch walks a list of matmul-free stages.
//
// A decoder stack at batch 1 is a stream of small sign matrices (1-6 MB each) and a 4096x4096 layer
// is worth 0.3 us of HBM time, so launching one kernel per stage (as the reference does,
// src/nanoquant/kernel/cuda/gemv_kernel.cu:406-425: two launches per linear) leaves the memory system
// idle most of the time.  Here the grid is sized to the machine once (one workgroup per CU, all
// co-resident) and every workgroup walks the same stage table:
//   * the sign words of a stage do not depend on any activation, so each lane issues its first
//     128-bit fetch of stage s before it waits for the producer of that stage's input;
//   * a stage whose input is produced by an earlier stage waits on that stage's completion counter
//     (one device-scope atomic per workgroup per stage), not on a kernel boundary; the host orders the
//     table so that independent work sits between a producer and its consumer;
//   * rows of a stage are split evenly over the workgroups; inside a workgroup the (row, 16-byte
//     unit) pairs are dealt round-robin to the 256 lanes, whatever the shape, and per-row sums are
//     finished with LDS float atomics.
// The arithmetic per 16-byte unit is the same as in nq_gemv.hip: sign pairs built with integer logic,
// v_dot2_f32_{f16,bf16} into fp32 accumulators, activations staged once per workgroup in LDS.
#include "nq_common.h"
#include "nq_kernels.h"

namespace nq {

constexpr int kStreamThreads = 256;
constexpr int kRowBlock = 128;                 // rows finished per pass of a workgroup
constexpr int kStreamLds = 144 * 1024;         // staged activations + row accumulators

__device__ __forceinline__ uint32_t comp_s(const uint4& v, int i) {
    return i == 0 ? v.x : i == 1 ? v.y : i == 2 ? v.z : v.w;
}

__device__ __forceinline__ uint4 load_unit(const RunStage& st, int row, int unit) {
    const uint32_t* p = st.bits + (size_t)row * st.words + 4 * unit;
    if (st.vec_bits) {
        typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
        const u32x4 v = __builtin_nontemporal_load((const u32x4*)p);
        return make_uint4(v.x, v.y, v.z, v.w);
    }
    uint4 w = make_uint4(0, 0, 0, 0);
    const int left = st.words - 4 * unit;
    w.x = p[0];
    if (left > 1) w.y = p[1];
    if (left > 2) w.z = p[2];
    if (left > 3) w.w = p[3];
    return w;
}

// Stage units [c0, c0+cu_n) of the (scaled) input into LDS; same layout as nq_gemv.hip:
// chunk (b, i, cu) at xs[(b*16 + i)*upad + cu] = columns 128*(c0+cu) + 8*i .. +7 as 16-bit values.
template <int DT, int BATCH>
__device__ __forceinline__ void stream_stage_input(uint4* xs, const RunStage& st, int c0, int cu_n, int upad) {
    using E = Elem<DT>;
    const int nchunks = cu_n * 16;
#pragma unroll 1
    for (int b = 0; b < BATCH; ++b) {
        for (int q = threadIdx.x; q < nchunks; q += kStreamThreads) {
            const int cu = q >> 4, i = q & 15;
            const int col = (c0 + cu) * 128 + i * 8;
            float v[8];
            if (st.vec_in && col + 8 <= st.K) {
                if (!st.in_f32) {
                    const uint16_t* xp = (const uint16_t*)st.in + (size_t)b * st.in_stride + col;
                    const uint4 xr = *(const uint4*)xp;
                    const uint4 sr = st.s_col ? *(const uint4*)(st.s_col + col)
                                              : make_uint4(E::kOnePair, E::kOnePair, E::kOnePair, E::kOnePair);
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const uint32_t xw = comp_s(xr, e), sw = comp_s(sr, e);
                        v[2 * e] = E::to_float(xw & 0xFFFFu) * E::to_float(sw & 0xFFFFu);
                        v[2 * e + 1] = E::to_float(xw >> 16) * E::to_float(sw >> 16);
                    }
                } else {
                    const float* hp = (const float*)st.in + (size_t)b * st.in_stride + col;
                    const float4 h0 = *(const float4*)hp, h1 = *(const float4*)(hp + 4);
                    v[0] = h0.x; v[1] = h0.y; v[2] = h0.z; v[3] = h0.w;
                    v[4] = h1.x; v[5] = h1.y; v[6] = h1.z; v[7] = h1.w;
                }
            } else {
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    const int c = col + e;
                    float t = 0.f;
                    if (c < st.K) {
                        if (!st.in_f32) {
                            t = E::to_float(((const uint16_t*)st.in)[(size_t)b * st.in_stride + c]);
                            if (st.s_col) t *= E::to_float(st.s_col[c]);
                        } else {
                            t = ((const float*)st.in)[(size_t)b * st.in_stride + c];
                        }
                    }
                    v[e] = t;
                }
            }
            uint4 p;
            p.x = (uint32_t)E::from_float(v[0]) | ((uint32_t)E::from_float(v[1]) << 16);
            p.y = (uint32_t)E::from_float(v[2]) | ((uint32_t)E::from_float(v[3]) << 16);
            p.z = (uint32_t)E::from_float(v[4]) | ((uint32_t)E::from_float(v[5]) << 16);
            p.w = (uint32_t)E::from_float(v[6]) | ((uint32_t)E::from_float(v[7]) << 16);
            xs[(b * 16 + i) * upad + cu] = p;
        }
    }
}

template <int DT, int BATCH>
__global__ __launch_bounds__(kStreamThreads) void gemv_stream_kernel(const RunStage* __restrict__ stages, int nstages,
                                                                     unsigned* counters, unsigned* status,
                                                                     unsigned spin_limit, int chunk_cap) {
    using E = Elem<DT>;
    extern __shared__ uint4 lds_raw[];
    float* racc = (float*)lds_raw;                              // [kRowBlock][BATCH]
    uint4* xs = lds_raw + (kRowBlock * BATCH * sizeof(float)) / sizeof(uint4);
    __shared__ int s_abort;
    const int tid = threadIdx.x;
    const unsigned nwg = gridDim.x, wg = blockIdx.x;
    if (tid == 0) s_abort = 0;
    __syncthreads();

#pragma unroll 1
    for (int s = 0; s < nstages; ++s) {
        const RunStage st = stages[s];
        const int r_begin = (int)(((long long)st.rows * wg) / nwg);
        const int r_end = (int)(((long long)st.rows * (wg + 1)) / nwg);
        const int chunk_units = min(st.units, chunk_cap);
        const int upad = chunk_units | 1;
        const int step_row = kStreamThreads / st.units, step_cu = kStreamThreads % st.units;  // for full-K chunks

        // First fetch of this stage, issued before any wait: the weights are always ready.
        uint4 wnext = make_uint4(0, 0, 0, 0);
        {
            const int nr0 = min(r_end - r_begin, kRowBlock);
            const int cu_n0 = chunk_units;
            if (tid < nr0 * cu_n0) wnext = load_unit(st, r_begin + tid / cu_n0, tid % cu_n0);
        }

        if (st.dep >= 0 || st.dep2 >= 0) {
            if (tid == 0 && !s_abort) {
                unsigned spins = 0;
#pragma unroll 1
                for (int which = 0; which < 2 && !s_abort; ++which) {
                    const int d = which ? st.dep2 : st.dep;
                    if (d < 0) continue;
                    while (__hip_atomic_load(counters + d, __ATOMIC_ACQUIRE, __HIP_MEMORY_SCOPE_AGENT) < nwg) {
                        __builtin_amdgcn_s_sleep(2);
                        if (++spins > spin_limit ||
                            __hip_atomic_load(status, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)) {
                            atomicOr(status, 1u);   // bounded wait: give up, flag it, let every workgroup drain
                            s_abort = 1;
                            break;
                        }
                    }
                }
            }
            __syncthreads();
        }
        const bool aborted = s_abort != 0;   // uniform: written before the barrier above or at entry

#pragma unroll 1
        for (int rb = r_begin; rb < r_end && !aborted; rb += kRowBlock) {
            const int nr = min(r_end - rb, kRowBlock);
            __syncthreads();                                   // previous users of racc / xs are done
            for (int i = tid; i < nr * BATCH; i += kStreamThreads) racc[i] = 0.f;
#pragma unroll 1
            for (int c0 = 0; c0 < st.units; c0 += chunk_units) {
                const int cu_n = min(chunk_units, st.units - c0);
                if (c0) __syncthreads();
                stream_stage_input<DT, BATCH>(xs, st, c0, cu_n, upad);
                __syncthreads();
                const int total = nr * cu_n;
                int f = tid;
                int row_l = tid / cu_n, cu = tid % cu_n;
                const int srow = (cu_n == st.units) ? step_row : kStreamThreads / cu_n;
                const int scu = (cu_n == st.units) ? step_cu : kStreamThreads % cu_n;
                const bool first_pass = (rb == r_begin && c0 == 0);
#pragma unroll 1
                for (; f - tid < total; f += kStreamThreads) {
                    uint4 w;
                    if (first_pass && f == tid) w = wnext;
                    else w = (f < total) ? load_unit(st, rb + row_l, c0 + cu) : make_uint4(0, 0, 0, 0);
                    if (f < total) {
                        float acc[BATCH];
#pragma unroll
                        for (int b = 0; b < BATCH; ++b) acc[b] = 0.f;
#pragma unroll
                        for (int wi = 0; wi < 4; ++wi) {
                            const uint32_t word = comp_s(w, wi);
                            uint32_t sp[16];
#pragma unroll
                            for (int j = 0; j < 16; ++j) sp[j] = ((word << j) & kSignPair) | E::kOnePair;
#pragma unroll
                            for (int b = 0; b < BATCH; ++b) {
                                uint4 xv[4];
#pragma unroll
                                for (int q = 0; q < 4; ++q) xv[q] = xs[(b * 16 + 4 * wi + q) * upad + cu];
#pragma unroll
                                for (int j = 0; j < 16; ++j) acc[b] = E::dot2(comp_s(xv[j >> 2], j & 3), sp[j], acc[b]);
                            }
                        }
#pragma unroll
                        for (int b = 0; b < BATCH; ++b) atomicAdd(&racc[row_l * BATCH + b], acc[b]);
                    }
                    row_l += srow;
                    cu += scu;
                    if (cu >= cu_n) { cu -= cu_n; ++row_l; }
                }
            }
            __syncthreads();
            for (int i = tid; i < nr * BATCH; i += kStreamThreads) {
                const int row = rb + i / BATCH, b = i % BATCH;
                float v = racc[i];
                if (st.s_row) v *= E::to_float(st.s_row[row]);
                const size_t o = (size_t)b * st.out_stride + row;
                if (st.addend) v += st.addend[o];
                if (st.out_f32) ((float*)st.out)[o] = v;
                else ((uint16_t*)st.out)[o] = E::from_float_clamped(v);
            }
        }

        if (st.signal) {
            __syncthreads();                                   // all of this workgroup's stores are issued
            if (tid == 0) __hip_atomic_fetch_add(counters + s, 1u, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_AGENT);
        }
    }

    // The last workgroup to leave puts the counters back to zero for the next launch; every other
    // workgroup has finished all of its waits by the time it bumped the exit counter.
    __syncthreads();
    if (tid == 0) {
        const unsigned done = __hip_atomic_fetch_add(counters + nstages, 1u, __ATOMIC_ACQ_REL, __HIP_MEMORY_SCOPE_AGENT);
        s_abort = (done == nwg - 1) ? 2 : 0;
    }
    __syncthreads();
    if (s_abort == 2) {
        for (int i = tid; i <= nstages; i += kStreamThreads)
            __hip_atomic_store(counters + i, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
}

// ---- host side --------------------------------------------------------------------------------
template <int DT, int BATCH>
static hipError_t launch_stream(const RunStage* stages, int nstages, unsigned* counters, unsigned* status,
                                int nwg, hipStream_t stream) {
    auto kern = gemv_stream_kernel<DT, BATCH>;
    static bool attr_done = false;
    if (!attr_done) {
        hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, kStreamLds);
        if (e != hipSuccess) return e;
        attr_done = true;
    }
    const int racc_bytes = kRowBlock * BATCH * (int)sizeof(float);
    int chunk_cap = (kStreamLds - racc_bytes) / (BATCH * 16 * (int)sizeof(uint4));
    chunk_cap = (chunk_cap - 1) & ~1;
    // LDS actually needed: the largest stage decides; the caller passes it through `lds_units`.
    hipLaunchKernelGGL(kern, dim3(nwg), dim3(kStreamThreads), kStreamLds, stream, stages, nstages, counters, status,
                       (unsigned)(1u << 22), chunk_cap);
    return hipGetLastError();
}

int stream_max_workgroups() {
    int dev = 0, cus = 0;
    if (hipGetDevice(&dev) != hipSuccess) return 0;
    if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) return 0;
    return cus;  // one 144 KB-LDS workgroup per CU: co-resident by construction on an idle device
}

hipError_t gemv_stream(int dtype, int batch, const RunStage* stages, int nstages, unsigned* counters,
                       unsigned* status, int nwg, hipStream_t stream) {
#define NQ_STREAM_CASE(B)                                                                              \
    case B:                                                                                            \
        return dtype == 0 ? launch_stream<0, B>(stages, nstages, counters, status, nwg, stream)       \
                          : launch_stream<1, B>(stages, nstages, counters, status, nwg, stream);
    switch (batch) {
        NQ_STREAM_CASE(1)
        NQ_STREAM_CASE(2)
        NQ_STREAM_CASE(4)
        NQ_STREAM_CASE(8)
        NQ_STREAM_CASE(16)
        default: return hipErrorInvalidValue;
    }
#undef NQ_STREAM_CASE
}

}  // namespace nq
