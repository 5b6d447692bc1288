// Decode path, run-list form: ONE launch covers a whole list of matmul-free stages.
//
// A decoder stack at batch 1 is a stream of small sign matrices (1-6 MB each) and a 4096x4096 layer
// is worth 0.3 us of HBM time, so launching one kernel per stage (as the reference does,
// src/nanoquant/kernel/cuda/gemv_kernel.cu:406-425: two launches per linear) leaves the memory system
// idle most of the time.  Here the grid is the concatenation of the work items of all stages, in an
// order in which every stage comes after the stages it depends on:
//   * a work item is one block of rows of one stage; items of different stages are in flight on the
//     same CU at the same time, so the latency of one (fetch, staging, hand-over) is covered by the
//     arithmetic of the others -- occupancy does the software pipelining;
//   * the sign words of an item do not depend on any activation, so each lane issues its first
//     128-bit fetch before the item waits for the producer of its input;
//   * an item whose input is produced by an earlier stage waits on that stage's completion counter
//     (device-scope atomics), not on a kernel boundary.  Workgroups are dispatched in index order, so a
//     waiting workgroup only ever waits for workgroups that are already running or done; the wait is
//     bounded all the same and an expiry is reported through the status word;
//   * inside a workgroup the (row, 16-byte unit) pairs are dealt round-robin to the 256 lanes,
//     whatever the shape, and per-row sums are finished with LDS float atomics.
// The arithmetic per 16-byte unit is the same as in nq_gemv.hip: sign pairs built with integer logic,
// v_dot2_f32_{f16,bf16} into fp32 accumulators, activations staged once per workgroup in LDS.
#include "nq_decode.h"
#include "nq_kernels.h"

// Development aid, never defined in the product build: per-workgroup phase timestamps.
#ifdef NQ_TRACE
#include <stdio.h>
#include <stdlib.h>
#include <vector>
__device__ unsigned long long* g_nq_trace = nullptr;
#define NQ_MARK(k) do { if (g_nq_trace && threadIdx.x == 0) g_nq_trace[(size_t)blockIdx.x * 8 + (k)] = __builtin_amdgcn_s_memtime(); } while (0)
#else
#define NQ_MARK(k) do { } while (0)
#endif

namespace nq {

constexpr int kStreamThreads = 256;
constexpr int kRowBlock = 128;                 // rows finished per pass of a workgroup
// Same-address device-scope atomics serialise at the memory side (tens of ns each), so completion
// counts are spread over kSubCounters addresses per stage and kExitSubs addresses for the exit count.
constexpr int kSubCounters = 8;
constexpr int kExitSubs = 64;
constexpr int kCounterStride = 8;              // 64-bit words between sub-counters: one 64-byte line each
// Counters are 64-bit and only ever grow: launch number g of a run list finds every exit sub-counter k
// in [g*members_k, (g+1)*members_k) for as long as the reading workgroup itself has not left, so
// g = value / members_k needs no reset between launches and no atomic that returns a value; stage s
// is complete in launch g when its sub-counters add up to (g+1) * wg_count(s).
constexpr int kStreamLdsMax = 144 * 1024;      // staged activations + row accumulators, upper bound

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

template <int DT, int BATCH>
__global__ __launch_bounds__(kStreamThreads) void gemv_stream_kernel(const RunStage* __restrict__ stages, int nstages,
                                                                     const int* __restrict__ wg_stage,
                                                                     unsigned long long* counters, unsigned* status,
                                                                     unsigned spin_limit, int chunk_cap) {
    using E = Elem<DT>;
    extern __shared__ uint4 lds_raw[];
    float* racc = (float*)lds_raw;                              // [kRowBlock][BATCH] row sums
    float* xsum = racc + kRowBlock * BATCH;                     // [BATCH][kXsumStride] per-unit input sums
    uint4* xs = lds_raw + ((kRowBlock + kXsumStride) * BATCH * sizeof(float)) / sizeof(uint4);
    __shared__ int s_flag;
    const int tid = threadIdx.x;
    const int wg = blockIdx.x;

    NQ_MARK(0);
    const int s = wg_stage[wg];
    const RunStage st = stages[s];
    const int rb = (wg - st.wg_begin) * st.rows_item;
    const int nr = min(st.rows - rb, st.rows_item);
    const int chunk_units = min(st.units, chunk_cap);
    const int upad = chunk_units | 1;
    StageInput sin;
    sin.in = st.in; sin.s_col = st.s_col; sin.K = st.K; sin.in_stride = st.in_stride;
    sin.in_f32 = st.in_f32; sin.in_coherent = st.in_coherent; sin.vec_in = st.vec_in;

    NQ_MARK(1);
    // First fetch, issued before any wait: the weights are always ready.
    uint4 wnext = make_uint4(0, 0, 0, 0);
    if (tid < nr * chunk_units) wnext = load_unit(st, rb + tid / chunk_units, tid % chunk_units);
    if (tid == 0) s_flag = 0;
    for (int i = tid; i < nr * BATCH; i += kStreamThreads) racc[i] = 0.f;

    // The row scale is needed last; fetch it first.
    float srow = 1.f;
    if (st.s_row && tid < nr) srow = E::to_float(st.s_row[rb + tid]);

    if (st.dep >= 0 || st.dep2 >= 0) {
        if (tid < kWave) {                                   // wavefront 0 polls; lanes 0..7 own one sub-counter each
            // which launch of this run list is this?  (see the note at kCounterStride)
            const unsigned long long* exit_sub = counters + (size_t)nstages * kSubCounters * kCounterStride;
            const unsigned total = gridDim.x;
            const unsigned sub = (unsigned)wg & (kExitSubs - 1);
            const unsigned members = (total + kExitSubs - 1 - sub) / kExitSubs;
            const unsigned long long gen =
                __hip_atomic_load(exit_sub + (size_t)sub * kCounterStride, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) / members;
            unsigned spins = 0;
            bool bad = false;
#pragma unroll 1
            for (int which = 0; which < 2 && !bad; ++which) {
                const int d = which ? st.dep2 : st.dep;
                if (d < 0) continue;
                const unsigned long long want = (gen + 1) * (unsigned long long)stages[d].wg_count;
                while (true) {
                    unsigned long long c = 0;
                    if (tid < kSubCounters)
                        c = __hip_atomic_load(counters + ((size_t)d * kSubCounters + tid) * kCounterStride, __ATOMIC_RELAXED,
                                              __HIP_MEMORY_SCOPE_AGENT);
                    c += __shfl_xor(c, 1, kWave);
                    c += __shfl_xor(c, 2, kWave);
                    c += __shfl_xor(c, 4, kWave);
                    const unsigned long long sum0 = __shfl(c, 0, kWave);
                    if (sum0 >= want) break;
                    __builtin_amdgcn_s_sleep(16);   // ~0.5 us between polls: pollers must not crowd out the producers
                    unsigned flagged = 0;
                    if (tid == 0) flagged = __hip_atomic_load(status, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    flagged = __shfl(flagged, 0, kWave);
                    if (++spins > spin_limit || flagged) {
                        if (tid == 0) atomicOr(status, 1u);   // bounded wait: give up, flag it, let the grid drain
                        bad = true;
                        break;
                    }
                }
            }
            if (bad && tid == 0) s_flag = 1;
            // 16-bit input written by another stage of this launch: ordinary loads follow, so the
            // caches of this CU / XCD have to drop what they hold (rare; h and addend never need it).
            if (st.heavy_acquire && tid == 0) __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
        }
    }
    __syncthreads();
    NQ_MARK(2);
    const bool aborted = s_flag != 0;

    if (!aborted) {
#pragma unroll 1
        for (int c0 = 0; c0 < st.units; c0 += chunk_units) {
            const int cu_n = min(chunk_units, st.units - c0);
            if (c0) __syncthreads();
            stage_units<DT, BATCH>(xs, xsum, sin, c0, cu_n, upad, kStreamThreads);
            __syncthreads();
            NQ_MARK(3);
            const int total = nr * cu_n;
            int row_l = tid / cu_n, cu = tid % cu_n;
            const int srow = kStreamThreads / cu_n, scu = kStreamThreads % cu_n;
            uint4 w = wnext;                                   // chunk 0: fetched before the wait
            if (c0 != 0 && tid < total) w = load_unit(st, rb + row_l, c0 + cu);
#pragma unroll 1
            for (int f = tid; f < total; f += kStreamThreads) {
                // next unit of this lane: put its fetch in flight before the arithmetic
                int nrow = row_l + srow, ncu = cu + scu;
                if (ncu >= cu_n) { ncu -= cu_n; ++nrow; }
                uint4 wpre = make_uint4(0, 0, 0, 0);
                if (f + kStreamThreads < total) wpre = load_unit(st, rb + nrow, c0 + ncu);

                float part[BATCH];
                UnitDot<DT, BATCH>::run(w, xs, xsum, upad, cu, part);
#pragma unroll
                for (int b = 0; b < BATCH; ++b) atomicAdd(&racc[row_l * BATCH + b], part[b]);
                w = wpre;
                row_l = nrow;
                cu = ncu;
            }
        }
        __syncthreads();
        NQ_MARK(4);
        for (int i = tid; i < nr * BATCH; i += kStreamThreads) {
            const int row = rb + i / BATCH, b = i % BATCH;
            float v = racc[i];
            if (BATCH == 1 && i < kStreamThreads) v *= srow;             // i == tid on the first trip
            else if (st.s_row) v *= E::to_float(st.s_row[row]);
            const size_t o = (size_t)b * st.out_stride + row;
            if (st.addend) {
                if (st.dep2 >= 0)
                    v += __builtin_bit_cast(float, __hip_atomic_load((const uint32_t*)st.addend + o, __ATOMIC_RELAXED,
                                                                     __HIP_MEMORY_SCOPE_AGENT));
                else
                    v += st.addend[o];
            }
            if (st.out_f32) {
                // fp32 results (h, partial sums over terms) may be read by other workgroups of this
                // launch: device-coherent store, completed before the counter below is bumped
                if (st.signal) __hip_atomic_store((uint32_t*)st.out + o, __builtin_bit_cast(uint32_t, v), __ATOMIC_RELAXED,
                                                  __HIP_MEMORY_SCOPE_AGENT);
                else ((float*)st.out)[o] = v;
            } else {
                ((uint16_t*)st.out)[o] = E::from_float_clamped(v);
            }
        }
    }

    // Workgroup-scope release + barrier: every lane's stores above have been acknowledged.
    NQ_MARK(5);
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    __syncthreads();
    NQ_MARK(6);
    if (tid == 0) {
        if (st.signal) {
            unsigned long long* c = counters + ((size_t)s * kSubCounters + (wg & (kSubCounters - 1))) * kCounterStride;
            if (st.heavy_release) __hip_atomic_fetch_add(c, 1ull, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_AGENT);
            else __hip_atomic_fetch_add(c, 1ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        unsigned long long* exit_sub = counters + (size_t)nstages * kSubCounters * kCounterStride;
        __hip_atomic_fetch_add(exit_sub + (size_t)(wg & (kExitSubs - 1)) * kCounterStride, 1ull, __ATOMIC_RELAXED,
                               __HIP_MEMORY_SCOPE_AGENT);
    }
    NQ_MARK(7);
}

size_t stream_counter_bytes(int nstages) { return ((size_t)nstages * kSubCounters + kExitSubs) * kCounterStride * sizeof(unsigned long long); }

// ---- host side --------------------------------------------------------------------------------
template <int DT, int BATCH>
static hipError_t launch_stream(const RunStage* stages, int nstages, const int* wg_stage, unsigned long long* counters,
                                unsigned* status, int total_wgs, int max_units, hipStream_t stream) {
    auto kern = gemv_stream_kernel<DT, BATCH>;
    const int racc_bytes = (kRowBlock + kXsumStride) * BATCH * (int)sizeof(float);
    int chunk_cap = (kStreamLdsMax - racc_bytes) / (BATCH * 16 * (int)sizeof(uint4));
    chunk_cap = (chunk_cap - 1) & ~1;
    if (chunk_cap > kXsumStride - 2) chunk_cap = kXsumStride - 2;
    const int chunk_units = max_units < chunk_cap ? max_units : chunk_cap;
    const size_t lds = (size_t)racc_bytes + (size_t)BATCH * 16 * (chunk_units | 1) * sizeof(uint4);
    static bool attr_done = false;
    if (lds > 64 * 1024 && !attr_done) {
        hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, kStreamLdsMax);
        if (e != hipSuccess) return e;
        attr_done = true;
    }
#ifdef NQ_TRACE
    static unsigned long long* tbuf = nullptr;
    static int calls = 0;
    if (getenv("NQ_TS") && !tbuf) {
        (void)hipMalloc(&tbuf, (size_t)total_wgs * 64);
        (void)hipMemcpyToSymbol(HIP_SYMBOL(g_nq_trace), &tbuf, sizeof(tbuf));
    }
#endif
    hipLaunchKernelGGL(kern, dim3(total_wgs), dim3(kStreamThreads), lds, stream, stages, nstages, wg_stage, counters,
                       status, (unsigned)(1u << 20), chunk_cap);
#ifdef NQ_TRACE
    if (tbuf && ++calls == 40) {
        (void)hipStreamSynchronize(stream);
        std::vector<unsigned long long> h((size_t)total_wgs * 8);
        (void)hipMemcpy(h.data(), tbuf, h.size() * 8, hipMemcpyDeviceToHost);
        std::vector<int> map(total_wgs);
        (void)hipMemcpy(map.data(), wg_stage, (size_t)total_wgs * 4, hipMemcpyDeviceToHost);
        FILE* f = fopen(getenv("NQ_TS"), "w");
        for (int i = 0; i < total_wgs; ++i) {
            fprintf(f, "%d %d", i, map[i]);
            for (int k = 0; k < 8; ++k) fprintf(f, " %llu", h[(size_t)i * 8 + k]);
            fprintf(f, "\n");
        }
        fclose(f);
    }
#endif
    return hipGetLastError();
}

// Rows per work item: about three 16-byte units per lane (measured best for a single decoder layer per
// launch: shorter items finish the first stages sooner), at most kRowBlock rows.
int stream_rows_per_item(int units) {
    int rows = (3 * kStreamThreads + units / 2) / units;
    if (rows < 1) rows = 1;
    if (rows > kRowBlock) rows = kRowBlock;
    return rows;
}

hipError_t gemv_stream(int dtype, int batch, const RunStage* stages, int nstages, const int* wg_stage,
                       unsigned long long* counters, unsigned* status, int total_wgs, int max_units, hipStream_t stream) {
#define NQ_STREAM_CASE(B)                                                                                          \
    case B:                                                                                                        \
        return dtype == 0                                                                                          \
                   ? launch_stream<0, B>(stages, nstages, wg_stage, counters, status, total_wgs, max_units, stream)  \
                   : launch_stream<1, B>(stages, nstages, wg_stage, counters, status, total_wgs, max_units, stream);
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
