// Shared device code of the matmul-free decode stages: staging of the (scaled) input vector in LDS
// and the arithmetic of one 16-byte unit of packed signs (4 words = 128 columns of one row).
//
// LDS layout of the staged input (per batch row b): 16-byte chunk (b, i, cu) at
// xs[xs_chunk(b, i, upad, cu)] = xs[b*(16*upad+1) + i*upad + cu] holds the 8 consecutive columns 128*(c0+cu) + 8*i .. +7 as 16-bit values;
// upad is odd.  For a fixed i the lanes of a row read consecutive chunks (conflict-free) and lanes of
// different rows read the same chunk (broadcast).  xsum[b*upad + cu] is the fp32 sum of the 128
// staged values of unit cu.
//
// Arithmetic, fp16.  The packed "half2" order puts the signs of the element pair j (j = 0..15) of a
// word at bits 15-j and 31-j, i.e. at the same position of both 16-bit halves.  A 16-bit pattern with
// only bit p set is itself a valid fp16 number when p is one of the exponent bits 10..14: its value
// is 2^-14, 2^-13, 2^-11, 2^-7, 2^+1.  So `word & mask_p` IS the operand pair (b_lo*c_p, b_hi*c_p)
// with b the packed bits, and one v_dot2_f32_f16 adds c_p * (b_lo*x_lo + b_hi*x_hi) to an fp32
// accumulator of class p.  Three shifted copies of the word (>>1, <<5, <<10) bring every one of the
// 16 pair positions onto an exponent bit, which makes 3 shifts + 16 ANDs + 16 dot2 per word instead
// of a shift, a mask and an OR per pair.  All scalings are powers of two and the products of two fp16
// numbers are exact in fp32, so sum_c acc_c / c_p = sum b*x exactly as accumulated, and the signed
// sum follows from  sum (1-2b) x = sum x - 2 sum b x  with sum x taken from xsum.
//
// bf16 has no such luck (its single exponent bits reach 2^-126, which underflows fp32 products), so
// the bf16 path keeps the +-1 operand: ((word << j) & 0x80008000) | (1.0, 1.0).
#pragma once
#include "nq_common.h"

namespace nq {

constexpr int kXsumStride = 576;   // floats of unit sums per batch row: >= largest staged chunk (| 1), multiple of 4

__device__ __forceinline__ uint32_t comp_d(const uint4& v, int i) {
    return i == 0 ? v.x : i == 1 ? v.y : i == 2 ? v.z : v.w;
}

// Description of a stage input as the staging code sees it.
struct StageInput {
    const void* in;         // [batch, in_stride]
    const uint16_t* s_col;  // per-column scale for 16-bit input, may be null
    int K, in_stride;
    int in_f32;             // input is fp32 (the intermediate h) instead of the 16-bit activation type
    int in_coherent;        // fp32 input written by other workgroups of the same launch
    int vec_in;             // 16-byte loads allowed
};

typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));

// By value on purpose: __builtin_bit_cast applied directly to a vector element (v.y, v[e]) reads
// element 0 with this compiler.
__device__ __forceinline__ float as_float(uint32_t bits) { return __builtin_bit_cast(float, bits); }
__device__ __forceinline__ uint32_t as_bits(float v) { return __builtin_bit_cast(uint32_t, v); }

// Raw buffer view (gfx9 resource words) of `bytes` bytes at p: loads past the end return zeros, so a
// lane whose columns lie beyond K is pointed past the end instead of being branched around.
__device__ __forceinline__ __amdgpu_buffer_rsrc_t raw_buffer(const void* p, uint32_t bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), 0, (int)bytes, 0x00020000);
}
constexpr uint32_t kPastEnd = 0x7FFFFFF0u;
constexpr int kCacheDefault = 0;
constexpr int kCacheAgentCoherent = 16;   // sc1: served coherently at device scope, not from this XCD's L2

// Two LDS layouts of a staged unit (128 columns = 64 pairs P = 0..63, pair P = columns 2P, 2P+1):
//   chunk-major (PM = false): 16-byte chunk i = P >> 2 holds pairs 4i..4i+3 = 8 consecutive columns;
//   pair-major  (PM = true):  16-byte chunk j = P & 15 holds pair j of each of the four 32-column words
//                             (dword wi = P >> 4), the order in which one sign-bit position of the
//                             four words of a unit addresses the columns; chunks are stored unit by unit.
// Returns the dword index into xs.
// 16-byte chunk index of (batch row b, chunk i, unit cu).  The batch-row pitch 16*upad + 1 chunks is
// 4 dwords off a multiple of 64: the 16 lanes of an MFMA operand read that differ only in the batch row
// fall into 16 different bank groups (a pitch of 16*upad chunks puts all of them into the same one).
__device__ __forceinline__ int xs_chunk(int b, int i, int upad, int cu) { return b * (16 * upad + 1) + i * upad + cu; }
// chunks of staged input for `batch` rows
__host__ __device__ constexpr int xs_chunks(int batch, int upad) { return batch * (16 * upad + 1); }

// Pair-major chunks are stored unit by unit (chunk j of unit cu at b*pitch + 16*cu + j): the 16 reads of
// one unit differ by compile-time offsets.
__device__ __forceinline__ int xs_chunk_pm(int b, int j, int upad, int cu) { return b * (16 * upad + 1) + 16 * cu + j; }

template <bool PM>
__device__ __forceinline__ int xs_dword(int b, int P, int upad, int cu) {
    if constexpr (PM) return xs_chunk_pm(b, P & 15, upad, cu) * 4 + (P >> 4);
    else return xs_chunk(b, P >> 2, upad, cu) * 4 + (P & 3);
}

// Stores the 8 consecutive 16-bit values r[0..7] of chunk i (columns 8i..8i+7) of unit cu.
template <bool PM>
__device__ __forceinline__ void store_chunk(uint4* xs, int b, int i, int upad, int cu, const uint16_t (&r)[8]) {
    if constexpr (PM) {
        uint32_t* xd = (uint32_t*)xs;
#pragma unroll
        for (int k = 0; k < 4; ++k) xd[xs_dword<true>(b, 4 * i + k, upad, cu)] = (uint32_t)r[2 * k] | ((uint32_t)r[2 * k + 1] << 16);
    } else {
        uint4 pk;
        pk.x = (uint32_t)r[0] | ((uint32_t)r[1] << 16);
        pk.y = (uint32_t)r[2] | ((uint32_t)r[3] << 16);
        pk.z = (uint32_t)r[4] | ((uint32_t)r[5] << 16);
        pk.w = (uint32_t)r[6] | ((uint32_t)r[7] << 16);
        xs[xs_chunk(b, i, upad, cu)] = pk;
    }
}

// The same with the 8 values as 4 packed pairs.
template <bool PM>
__device__ __forceinline__ void store_chunk_packed(uint4* xs, int b, int i, int upad, int cu, const uint32_t (&rp)[4]) {
    if constexpr (PM) {
        uint32_t* xd = (uint32_t*)xs;
#pragma unroll
        for (int k = 0; k < 4; ++k) xd[xs_dword<true>(b, 4 * i + k, upad, cu)] = rp[k];
    } else {
        xs[xs_chunk(b, i, upad, cu)] = make_uint4(rp[0], rp[1], rp[2], rp[3]);
    }
}

// Staging variants below: `xsum` (may be null) receives the per-unit sums, `xtot` (may be null) the sum over all staged units per batch row
// (LDS float atomics; the caller zeroes it and puts a barrier before and after).

// it / n for 0 <= it < 2^23 with rcp = 1.f / n: the float product is off by one at most (the compiler's exact 32-bit
// division costs some 25 lane instructions, as much as the rest of a staged chunk).
__device__ __forceinline__ int small_div(int it, int n, float rcp) {
    int q = (int)((float)it * rcp);
    const int r = it - q * n;
    if (r >= n) ++q;
    else if (r < 0) --q;
    return q;
}

// Coherent fp32 input (the intermediate h written by other workgroups of this launch): 16-byte
// device-coherent loads, kBurst per lane in flight before the first is consumed (a round trip to the
// memory side costs about a microsecond; 256 lanes x 4 loads cover 4096 values in one round trip).
// One lane holds 4 consecutive values = 2 pairs; the 128 values of a unit sit in 32 consecutive lanes.
// Requires K % 4 == 0 and 16-byte aligned rows.
template <int DT, int BATCH, bool PM>
__device__ __forceinline__ void stage_units_coherent(uint4* xs, float* xsum, float* xtot, const StageInput& st, int c0,
                                                     int cu_n, int upad, int nthreads) {
    using E = Elem<DT>;
    constexpr int kBurst = 4;
    const int nquads = cu_n * 32;
    const int total = BATCH * nquads;
    const __amdgpu_buffer_rsrc_t rsrc =
        raw_buffer(st.in, (uint32_t)(((size_t)(BATCH - 1) * st.in_stride + st.K) * sizeof(float)));
    const float rcp = 1.f / (float)nquads;
#pragma unroll 1
    for (int it0 = threadIdx.x; it0 < total; it0 += nthreads * kBurst) {   // wave-uniform trip count: it0 - lane
        u32x4_t raw[kBurst];
        int bq[kBurst];
#pragma unroll
        for (int j = 0; j < kBurst; ++j) {
            const int it = it0 + j * nthreads;
            const int b = small_div(it, nquads, rcp), q = it - b * nquads;
            bq[j] = b;
            const int col = c0 * 128 + 4 * q;
            const uint32_t off = (it < total && col < st.K) ? (uint32_t)(((size_t)b * st.in_stride + col) * sizeof(float)) : kPastEnd;
            raw[j] = __builtin_amdgcn_raw_buffer_load_b128(rsrc, off, 0, kCacheAgentCoherent);
        }
#pragma unroll
        for (int j = 0; j < kBurst; ++j) {
            const int it = it0 + j * nthreads;
            const int b = bq[j], q = it - b * nquads;
            const uint16_t r0 = E::from_float(as_float(raw[j].x));
            const uint16_t r1 = E::from_float(as_float(raw[j].y));
            const uint16_t r2 = E::from_float(as_float(raw[j].z));
            const uint16_t r3 = E::from_float(as_float(raw[j].w));
            // the sum of what the dot products will actually see; lanes past the end hold zeros
            const float tot = group_sum((E::to_float(r0) + E::to_float(r1)) + (E::to_float(r2) + E::to_float(r3)), 32);
            if (it < total) {
                const int cu = q >> 5, P = 2 * (q & 31);
                uint32_t* xd = (uint32_t*)xs;
                xd[xs_dword<PM>(b, P, upad, cu)] = (uint32_t)r0 | ((uint32_t)r1 << 16);
                xd[xs_dword<PM>(b, P + 1, upad, cu)] = (uint32_t)r2 | ((uint32_t)r3 << 16);
                if ((q & 31) == 0) {
                    if (xsum) xsum[b * upad + cu] = tot;
                    if (xtot) atomicAdd(&xtot[b], tot);
                }
            }
        }
    }
}

// 16-bit input (times its per-column scale) or non-coherent fp32 input, 8 columns per lane and load.
// Requires 16-byte aligned rows and K % 8 == 0 (st.vec_in).
template <int DT, int BATCH, bool PM>
__device__ __forceinline__ void stage_units_vector(uint4* xs, float* xsum, float* xtot, const StageInput& st, int c0,
                                                   int cu_n, int upad, int nthreads) {
    using E = Elem<DT>;
    constexpr int kBurst = 6;   // 256 lanes x 6 chunks = 12288 columns in one round trip
    const int nchunks = cu_n * 16;
    const int total = BATCH * nchunks;
    const uint32_t esize = st.in_f32 ? 4u : 2u;
    const __amdgpu_buffer_rsrc_t rin = raw_buffer(st.in, (uint32_t)(((size_t)(BATCH - 1) * st.in_stride + st.K) * esize));
    const bool scaled = !st.in_f32 && st.s_col != nullptr;
    const __amdgpu_buffer_rsrc_t rsc = raw_buffer(scaled ? (const void*)st.s_col : st.in, scaled ? (uint32_t)st.K * 2u : 0u);
    const float rcp = 1.f / (float)nchunks;
#pragma unroll 1
    for (int it0 = threadIdx.x; it0 < total; it0 += nthreads * kBurst) {
        u32x4_t raw_a[kBurst], raw_b[kBurst];
        int bq[kBurst];
#pragma unroll
        for (int j = 0; j < kBurst; ++j) {
            const int it = it0 + j * nthreads;
            const int b = small_div(it, nchunks, rcp), q = it - b * nchunks;
            bq[j] = b;
            const int col = c0 * 128 + 8 * q;
            const bool live = it < total && col < st.K;
            const uint32_t off = live ? (uint32_t)(((size_t)b * st.in_stride + col) * esize) : kPastEnd;
            raw_a[j] = __builtin_amdgcn_raw_buffer_load_b128(rin, off, 0, kCacheDefault);
            if (st.in_f32) raw_b[j] = __builtin_amdgcn_raw_buffer_load_b128(rin, live ? off + 16u : kPastEnd, 0, kCacheDefault);
            else raw_b[j] = __builtin_amdgcn_raw_buffer_load_b128(rsc, live ? (uint32_t)col * 2u : kPastEnd, 0, kCacheDefault);
        }
        // a wavefront whose 64 chunks of a burst slot all lie past the end skips the slot (wave-uniform branch)
        const int wave_first = __builtin_amdgcn_readfirstlane(it0 - (int)(threadIdx.x & 63));
#pragma unroll
        for (int j = 0; j < kBurst; ++j) {
            if (wave_first + j * nthreads >= total) continue;
            const int it = it0 + j * nthreads;
            const int b = bq[j], q = it - b * nchunks;
            if constexpr (DT == 0) {
                if (!st.in_f32) {
                    // fp16 input: packed products, rounded once to fp16 like the fp32 product below (the product of two
                    // fp16 numbers is exact in fp32), and their sum with the packed dot product: 8 lane operations per
                    // chunk instead of 50
                    typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
                    uint32_t rp[4];
                    float tot = 0.f;
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        half2_t xv = __builtin_bit_cast(half2_t, (uint32_t)raw_a[j][e]);
                        if (scaled) xv = xv * __builtin_bit_cast(half2_t, (uint32_t)raw_b[j][e]);
                        rp[e] = __builtin_bit_cast(uint32_t, xv);
                        tot = __builtin_amdgcn_fdot2(xv, (half2_t){(_Float16)1.f, (_Float16)1.f}, tot, false);
                    }
                    tot = group_sum(tot, 16);
                    if (it < total) {
                        const int cu = q >> 4, i = q & 15;
                        store_chunk_packed<PM>(xs, b, i, upad, cu, rp);
                        if (i == 0) {
                            if (xsum) xsum[b * upad + cu] = tot;
                            if (xtot) atomicAdd(&xtot[b], tot);
                        }
                    }
                    continue;
                }
            }
            float v[8];
            if (!st.in_f32) {
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const uint32_t xw = raw_a[j][e], sw = scaled ? raw_b[j][e] : E::kOnePair;
                    v[2 * e] = E::to_float(xw & 0xFFFFu) * E::to_float(sw & 0xFFFFu);
                    v[2 * e + 1] = E::to_float(xw >> 16) * E::to_float(sw >> 16);
                }
            } else {
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    v[e] = as_float(raw_a[j][e]);
                    v[4 + e] = as_float(raw_b[j][e]);
                }
            }
            uint16_t r[8];
            float tot = 0.f;
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                r[e] = E::from_float(v[e]);
                tot += E::to_float(r[e]);          // the sum of what the dot products will actually see
            }
            // the 16 chunks of a unit are held by 16 consecutive lanes: finish the unit sum with DPP
            tot = group_sum(tot, 16);
            if (it < total) {
                const int cu = q >> 4, i = q & 15;
                store_chunk<PM>(xs, b, i, upad, cu, r);
                if (i == 0) {
                    if (xsum) xsum[b * upad + cu] = tot;
                    if (xtot) atomicAdd(&xtot[b], tot);
                }
            }
        }
    }
}

// Element-wise fallback for inputs that allow no 16-byte loads (odd K, unaligned rows).
template <int DT, int BATCH, bool PM>
__device__ __forceinline__ void stage_units_scalar(uint4* xs, float* xsum, float* xtot, const StageInput& st, int c0,
                                                   int cu_n, int upad, int nthreads) {
    using E = Elem<DT>;
    const int nchunks = cu_n * 16;
#pragma unroll 1
    for (int b = 0; b < BATCH; ++b) {
#pragma unroll 1
        for (int q0 = 0; q0 < nchunks; q0 += nthreads) {    // all lanes take every trip: group_sum needs them
            const int q = q0 + threadIdx.x;
            const int cu = q >> 4, i = q & 15;
            const int col = (c0 + cu) * 128 + i * 8;
            uint16_t r[8];
            float tot = 0.f;
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const int c = col + e;
                float t = 0.f;
                if (q < nchunks && c < st.K) {
                    if (!st.in_f32) {
                        t = E::to_float(((const uint16_t*)st.in)[(size_t)b * st.in_stride + c]);
                        if (st.s_col) t *= E::to_float(st.s_col[c]);
                    } else if (st.in_coherent) {
                        t = __builtin_bit_cast(float, __hip_atomic_load((const uint32_t*)st.in + (size_t)b * st.in_stride + c,
                                                                        __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT));
                    } else {
                        t = ((const float*)st.in)[(size_t)b * st.in_stride + c];
                    }
                }
                r[e] = E::from_float(t);
                tot += E::to_float(r[e]);
            }
            tot = group_sum(tot, 16);
            if (q < nchunks) {
                store_chunk<PM>(xs, b, i, upad, cu, r);
                if (i == 0) {
                    if (xsum) xsum[b * upad + cu] = tot;
                    if (xtot) atomicAdd(&xtot[b], tot);
                }
            }
        }
    }
}

// Stage units [c0, c0+cu_n) for BATCH rows.  All threads of the workgroup call this; nthreads is the
// workgroup size (a multiple of 64).  Must be followed by a barrier before xs/xsum/xtot are read.
template <int DT, int BATCH, bool PM = false>
__device__ __forceinline__ void stage_units(uint4* xs, float* xsum, const StageInput& st, int c0, int cu_n, int upad,
                                            int nthreads, float* xtot = nullptr) {
    if (!st.vec_in || (st.K & 7)) stage_units_scalar<DT, BATCH, PM>(xs, xsum, xtot, st, c0, cu_n, upad, nthreads);
    else if (st.in_f32 && st.in_coherent) stage_units_coherent<DT, BATCH, PM>(xs, xsum, xtot, st, c0, cu_n, upad, nthreads);
    else stage_units_vector<DT, BATCH, PM>(xs, xsum, xtot, st, c0, cu_n, upad, nthreads);
}

// Staging for the run-list kernel's 16-bit arithmetic (pair-major layout, unit totals to unit_tot[b * upad + cu]):
// one lane takes the 8 columns of one 16-byte chunk for kRows batch rows.  The column scale is loaded once for all of
// them, every load of a lane is in flight before the first is used (an input of 4096 columns at batch 16 is one round
// trip to the memory side for the workgroup instead of two or three), and no index is divided.  A wavefront's 64
// chunks belong to one half of the batch rows (the chunk count is padded to a multiple of 64).  Requires 16-byte
// aligned rows and K % 8 == 0; everything else goes through stage_units.
template <int DT, int BATCH, int THREADS>
__device__ __forceinline__ void stage_units_rows(uint4* xs, float* unit_tot, const StageInput& st, int c0, int cu_n,
                                                 int upad) {
    if (!st.vec_in || (st.K & 7)) {
        stage_units<DT, BATCH, true>(xs, unit_tot, st, c0, cu_n, upad, THREADS, nullptr);
        return;
    }
    using E = Elem<DT>;
    constexpr int kParts = BATCH >= 8 ? 2 : 1;
    constexpr int kRows = BATCH / kParts;                    // batch rows per lane
    constexpr int kRowsF32 = kRows > 4 ? 4 : kRows;          // fp32 input: two loads per row, half as many rows in flight
    const int lane = threadIdx.x & 63;
    const int nchunks = cu_n * 16;
    const int npad = ((cu_n + 3) & ~3) * 16;
    const int nitems = kParts * npad;
    const uint32_t esize = st.in_f32 ? 4u : 2u;
    const __amdgpu_buffer_rsrc_t rin = raw_buffer(st.in, (uint32_t)(((size_t)(BATCH - 1) * st.in_stride + st.K) * esize));
    const bool scaled = !st.in_f32 && st.s_col != nullptr;
    const __amdgpu_buffer_rsrc_t rsc = raw_buffer(scaled ? (const void*)st.s_col : st.in, scaled ? (uint32_t)st.K * 2u : 0u);
    const uint32_t row_bytes = (uint32_t)st.in_stride * esize;
    // the 8 rounded values r of chunk (b, q) and their unit total
    auto put = [&](int b, int q, const uint32_t (&rp)[4], float tot) {
        tot = group_sum(tot, 16);                            // the 16 chunks of a unit sit in 16 consecutive lanes
        if (q < nchunks) {
            store_chunk_packed<true>(xs, b, q & 15, upad, q >> 4, rp);
            if ((q & 15) == 0) unit_tot[b * upad + (q >> 4)] = tot;
        }
    };
    auto round_and_put = [&](int b, int q, const float (&v)[8]) {
        uint32_t rp[4];
        float tot = 0.f;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            rp[e] = (uint32_t)E::from_float(v[2 * e]) | ((uint32_t)E::from_float(v[2 * e + 1]) << 16);
            tot = E::dot2(rp[e], E::kOnePair, tot);          // the sum of what the dot products will actually see
        }
        put(b, q, rp, tot);
    };
#pragma unroll 1
    for (int item = threadIdx.x; item - lane < nitems; item += THREADS) {     // wave-uniform trip count
        const int part = (kParts > 1 && item - lane >= npad) ? 1 : 0;           // wave-uniform
        const int q = item - part * npad, b0 = part * kRows;
        const int col = c0 * 128 + 8 * q;
        const bool live = q < nchunks && col < st.K;
        const uint32_t off0 = (uint32_t)b0 * row_bytes + (uint32_t)col * esize;
        if (!st.in_f32) {
            const u32x4_t sc = __builtin_amdgcn_raw_buffer_load_b128(rsc, live ? (uint32_t)col * 2u : kPastEnd, 0, kCacheDefault);
            u32x4_t raw[kRows];
#pragma unroll
            for (int j = 0; j < kRows; ++j)
                raw[j] = __builtin_amdgcn_raw_buffer_load_b128(rin, live ? off0 + (uint32_t)j * row_bytes : kPastEnd, 0, kCacheDefault);
#pragma unroll
            for (int j = 0; j < kRows; ++j) {
                if constexpr (DT == 0) {
                    // packed products, rounded once to fp16 (the product of two fp16 numbers is exact in fp32), and their
                    // sum with the packed dot product
                    typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
                    uint32_t rp[4];
                    float tot = 0.f;
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        half2_t xv = __builtin_bit_cast(half2_t, (uint32_t)raw[j][e]);
                        if (scaled) xv = xv * __builtin_bit_cast(half2_t, (uint32_t)sc[e]);
                        rp[e] = __builtin_bit_cast(uint32_t, xv);
                        tot = __builtin_amdgcn_fdot2(xv, (half2_t){(_Float16)1.f, (_Float16)1.f}, tot, false);
                    }
                    put(b0 + j, q, rp, tot);
                } else {
                    float v[8];
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const uint32_t xw = raw[j][e], sw = scaled ? sc[e] : E::kOnePair;
                        v[2 * e] = E::to_float(xw & 0xFFFFu) * E::to_float(sw & 0xFFFFu);
                        v[2 * e + 1] = E::to_float(xw >> 16) * E::to_float(sw >> 16);
                    }
                    round_and_put(b0 + j, q, v);
                }
            }
        } else {
#pragma unroll
            for (int j0 = 0; j0 < kRows; j0 += kRowsF32) {
                u32x4_t ra[kRowsF32], rb[kRowsF32];
#pragma unroll
                for (int j = 0; j < kRowsF32; ++j) {
                    const uint32_t off = live ? off0 + (uint32_t)(j0 + j) * row_bytes : kPastEnd;
                    if (st.in_coherent) {
                        ra[j] = __builtin_amdgcn_raw_buffer_load_b128(rin, off, 0, kCacheAgentCoherent);
                        rb[j] = __builtin_amdgcn_raw_buffer_load_b128(rin, live ? off + 16u : kPastEnd, 0, kCacheAgentCoherent);
                    } else {
                        ra[j] = __builtin_amdgcn_raw_buffer_load_b128(rin, off, 0, kCacheDefault);
                        rb[j] = __builtin_amdgcn_raw_buffer_load_b128(rin, live ? off + 16u : kPastEnd, 0, kCacheDefault);
                    }
                }
#pragma unroll
                for (int j = 0; j < kRowsF32; ++j) {
                    float v[8];
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        v[e] = as_float(ra[j][e]);
                        v[4 + e] = as_float(rb[j][e]);
                    }
                    round_and_put(b0 + j0 + j, q, v);
                }
            }
        }
    }
}

// Signed sum over one unit for BATCH rows: out[b] = sum_{c in unit} sgn(bit c) * x[b][c].
template <int DT, int BATCH>
struct UnitDot;

template <int BATCH>
struct UnitDot<0, BATCH> {   // fp16: single-exponent-bit operands, 5 accumulator classes
    static __device__ __forceinline__ void run(const uint4& w, const uint4* xs, const float* xsum, int upad, int cu,
                                               float (&out)[BATCH]) {
        using E = Elem<0>;
        constexpr uint32_t M14 = 0x40004000u, M13 = 0x20002000u, M12 = 0x10001000u, M11 = 0x08000800u, M10 = 0x04000400u;
        float a14[BATCH], a13[BATCH], a12[BATCH], a11[BATCH], a10[BATCH];
#pragma unroll
        for (int b = 0; b < BATCH; ++b) a14[b] = a13[b] = a12[b] = a11[b] = a10[b] = 0.f;
#pragma unroll
        for (int wi = 0; wi < 4; ++wi) {
            const uint32_t w0 = comp_d(w, wi);
            const uint32_t wa = w0 >> 1, wb = w0 << 5, wc = w0 << 10;
            // pair j -> (source, class): j=0 (wa,14); j=1..5 (w0,14..10); j=6..10 (wb,14..10); j=11..15 (wc,14..10)
            const uint32_t m0 = wa & M14;
            const uint32_t m1 = w0 & M14, m2 = w0 & M13, m3 = w0 & M12, m4 = w0 & M11, m5 = w0 & M10;
            const uint32_t m6 = wb & M14, m7 = wb & M13, m8 = wb & M12, m9 = wb & M11, m10 = wb & M10;
            const uint32_t m11 = wc & M14, m12 = wc & M13, m13 = wc & M12, m14 = wc & M11, m15 = wc & M10;
#pragma unroll
            for (int b = 0; b < BATCH; ++b) {
                const uint4 x0 = xs[xs_chunk(b, 4 * wi + 0, upad, cu)];
                const uint4 x1 = xs[xs_chunk(b, 4 * wi + 1, upad, cu)];
                const uint4 x2 = xs[xs_chunk(b, 4 * wi + 2, upad, cu)];
                const uint4 x3 = xs[xs_chunk(b, 4 * wi + 3, upad, cu)];
                a14[b] = E::dot2(x0.x, m0, a14[b]);
                a14[b] = E::dot2(x0.y, m1, a14[b]);
                a13[b] = E::dot2(x0.z, m2, a13[b]);
                a12[b] = E::dot2(x0.w, m3, a12[b]);
                a11[b] = E::dot2(x1.x, m4, a11[b]);
                a10[b] = E::dot2(x1.y, m5, a10[b]);
                a14[b] = E::dot2(x1.z, m6, a14[b]);
                a13[b] = E::dot2(x1.w, m7, a13[b]);
                a12[b] = E::dot2(x2.x, m8, a12[b]);
                a11[b] = E::dot2(x2.y, m9, a11[b]);
                a10[b] = E::dot2(x2.z, m10, a10[b]);
                a14[b] = E::dot2(x2.w, m11, a14[b]);
                a13[b] = E::dot2(x3.x, m12, a13[b]);
                a12[b] = E::dot2(x3.y, m13, a12[b]);
                a11[b] = E::dot2(x3.z, m14, a11[b]);
                a10[b] = E::dot2(x3.w, m15, a10[b]);
            }
        }
#pragma unroll
        for (int b = 0; b < BATCH; ++b) {
            // undo the class scalings (exact powers of two): 2^1, 2^-7, 2^-11, 2^-13, 2^-14
            const float bx = a14[b] * 0.5f + a13[b] * 128.f + a12[b] * 2048.f + a11[b] * 8192.f + a10[b] * 16384.f;
            out[b] = xsum[b * upad + cu] - 2.f * bx;
        }
    }
};

template <int BATCH>
struct UnitDot<1, BATCH> {   // bf16: +-1 operand pairs
    static __device__ __forceinline__ void run(const uint4& w, const uint4* xs, const float* xsum, int upad, int cu,
                                               float (&out)[BATCH]) {
        using E = Elem<1>;
        (void)xsum;
        constexpr int NACC = BATCH >= 4 ? 1 : 4;
        float acc[BATCH][NACC];
#pragma unroll
        for (int b = 0; b < BATCH; ++b)
#pragma unroll
            for (int a = 0; a < NACC; ++a) acc[b][a] = 0.f;
#pragma unroll
        for (int wi = 0; wi < 4; ++wi) {
            const uint32_t word = comp_d(w, wi);
            uint32_t sp[16];
#pragma unroll
            for (int j = 0; j < 16; ++j) sp[j] = ((word << j) & kSignPair) | E::kOnePair;
#pragma unroll
            for (int b = 0; b < BATCH; ++b) {
                uint4 xv[4];
#pragma unroll
                for (int q = 0; q < 4; ++q) xv[q] = xs[xs_chunk(b, 4 * wi + q, upad, cu)];
#pragma unroll
                for (int j = 0; j < 16; ++j)
                    acc[b][j % NACC] = E::dot2(comp_d(xv[j >> 2], j & 3), sp[j], acc[b][j % NACC]);
            }
        }
#pragma unroll
        for (int b = 0; b < BATCH; ++b) {
            float t = acc[b][0];
#pragma unroll
            for (int a = 1; a < NACC; ++a) t += acc[b][a];
            out[b] = t;
        }
    }
};

// ---- MFMA-assisted unit arithmetic (batch >= 4) -----------------------------------------------------
// One v_mfma_f32_16x16x32 multiplies a 16-row x 32-column block of +-1 (A operand) with 32 columns x
// 16 batch rows of staged activations (B operand).  Lane l of the wavefront owns matrix row l & 15 and
// the column octet l >> 4: its 16 bytes of sign words (one unit of ITS row) feed 16 MFMAs, one per
// (word, byte) of the unit, because the 8 signs a lane contributes to an MFMA are exactly one byte
// group of the "half2" order: bits (15-s, 31-s), s = 4*q + c, for the pairs c = 0..3 of quarter q.
// The four lanes that share a row hold four different units of that row, so a wavefront covers
// 16 rows x 4 units per fetch and the contraction index of an MFMA is "unit-of-the-lane x octet".
// The cost per packed bit does not depend on the batch size up to 16.
template <int DT>
struct Mfma16;
template <>
struct Mfma16<0> {
    static __device__ __forceinline__ float4_t run(uint4 a, uint4 b, float4_t c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8_t, a), __builtin_bit_cast(half8_t, b), c, 0, 0, 0);
    }
};
template <>
struct Mfma16<1> {
    static __device__ __forceinline__ float4_t run(uint4 a, uint4 b, float4_t c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf168_t, a), __builtin_bit_cast(bf168_t, b), c, 0, 0, 0);
    }
};

// The single-exponent-bit operand of the matmul-free loop as the MFMA weight operand.  A 16-bit pattern with only one
// exponent bit set is itself a number of the type: fp16 bits 14..10 = 2^1, 2^-7, 2^-11, 2^-13, 2^-14 (five classes);
// bf16 bits 14, 13, 12 = 2^1, 2^-63, 2^-95 (three classes: the lower exponent bits would put the products of small
// activations below the fp32 normal range).  For a pair position j the four dwords `word_wi & mask` (wi = 0..3) ARE the
// pairs c*(b_lo, b_hi) of pair j of the unit's four words with c the class constant of the mask bit: one AND per dword
// instead of a shift and a bit-field insert (and no inline assembly ahead of an MFMA: for instructions it does not
// know the compiler keeps no wait states, and a bit-field insert written that way gave wrong sums now and then).
// Shifted copies of every word bring all 16 pair positions onto a class bit: pair j sits at bits (15-j, 31-j); pair 0
// takes the copy >> 1 and class 0, pair j >= 1 the copy << C*((j-1)/C) and class (j-1) % C with C classes.  The
// activation operand comes from the pair-major staging layout, whose chunk j holds exactly those 8 columns.  Each
// class has its own accumulator; sum b*x = sum_c acc_c / c (pow2_combine), and the signed sum is
// (sum of x) - 2 (sum b*x).  Zero words contribute nothing, so "no unit" is w = 0.
template <int DT>
struct Pow2 {
    static constexpr int kClasses = DT == 0 ? 5 : 3;
};

template <int DT, int BATCH>
__device__ __forceinline__ void unit_mfma_pow2(const uint4& w, const uint4* xs, int upad, int cu,
                                               float4_t (&acc)[Pow2<DT>::kClasses]) {
    constexpr int C = Pow2<DT>::kClasses;
    constexpr uint32_t M14 = 0x40004000u;
    const int nb = min((int)(threadIdx.x & 15), BATCH - 1);
    const uint4* xrow = xs + xs_chunk_pm(nb, 0, upad, cu);
    {   // pair 0: bit 15 -> bit 14
        const uint4 a = make_uint4((w.x >> 1) & M14, (w.y >> 1) & M14, (w.z >> 1) & M14, (w.w >> 1) & M14);
        acc[0] = Mfma16<DT>::run(a, xrow[0], acc[0]);
    }
#pragma unroll
    for (int j0 = 1; j0 < 16; j0 += C) {
        const int sh = j0 - 1;                            // C * ((j - 1) / C) for the pairs j0 .. j0 + C - 1
        const uint32_t s0 = w.x << sh, s1 = w.y << sh, s2 = w.z << sh, s3 = w.w << sh;
#pragma unroll
        for (int cls = 0; cls < C; ++cls) {
            const int j = j0 + cls;
            if (j > 15) break;
            const uint32_t mask = M14 >> cls;
            const uint4 a = make_uint4(s0 & mask, s1 & mask, s2 & mask, s3 & mask);
            acc[cls] = Mfma16<DT>::run(a, xrow[j], acc[cls]);
        }
    }
}

// sum b*x per accumulator element from the class accumulators (exact power-of-two rescaling)
template <int DT>
__device__ __forceinline__ float4_t pow2_combine(const float4_t (&acc)[Pow2<DT>::kClasses]) {
    if constexpr (DT == 0) return acc[0] * 0.5f + acc[1] * 128.f + acc[2] * 2048.f + acc[3] * 8192.f + acc[4] * 16384.f;
    else return acc[0] * 0.5f + acc[1] * 0x1p63f + acc[2] * 0x1p95f;
}

// ---- one-bit fp4 weights x fp8 pieces of the input (batch 1..4, fp16 and bf16 alike) ---------------
// v_mfma_scale_f32_16x16x128_f8f6f4 takes an fp4 (e2m1) A operand, an fp8 (e4m3) B operand and one power-of-two
// scale per operand and block of 32 contraction indices.  The eight nibbles of a packed word are eight fp4 numbers,
// so the sign bits at position p of every nibble ("class" p, eight signs per word) become a weight operand with ONE
// lane operation:
//   p = 0, 1, 2:  w & (0x11111111 << p)            nibble = one-hot bit p = 0.5, 1, 2 times the packed bit b
//   p = 3:        (w & 0x88888888) | 0x22222222     nibble = sign bit b on the number 1.0 = +-1, i.e. 1 - 2 b
// Four lane operations per 32 signs, and one MFMA multiplies 16 rows x 512 columns of signs.  The signed sum over
// the columns of the classes 0..2 is (sum of u) - 2 (sum of b u): their input pieces are staged NEGATED and the
// block scale of the B operand carries the factors 4, 2, 1 that make every class contribute -2 b u, so that all four
// classes add into one accumulator; (sum of u) over the columns of classes 0..2 is taken once while staging (xtot).
//
// The input is staged as kQ8Pieces fp8 numbers per element, u = x * s * S ~ q0 + q1 + q2 with
// q_k = fp8(u - q_0 - .. - q_{k-1}) (round to nearest, residuals exact in fp32) and S the power of two that brings
// the largest |u| of the element's UNIT (128 consecutive columns) into [128, 256): one scale per unit and batch
// row, handed to the MFMA as its block scale, so an outlier lowers the resolution of its own 127 neighbours only.
// Every piece carries 4 significant bits; three reproduce u to 2^-12 relative or 2^-17 of the unit's maximum,
// whichever is larger (fp16 staging keeps 2^-11 relative).  Products are exact, accumulators fp32; the
// instruction's internal 128-term sum keeps 13 bits below its largest product (measured).  Pieces and batch rows
// are columns of the B operand: column j = b * kQ8Pieces + piece, at most 16.
//
// Operand geometry (measured on gfx950 with one-hot operands): lane (i = l & 15, g = l >> 4) supplies
//   A (fp4, 4 dwords): row i, k = 32 g + idx, idx = 8 t + e for nibble e of dword t;
//   B (fp8, 8 dwords): column i, k = 64 (idx >> 4) + 16 g + (idx & 15) for byte idx of the 32;
//   B block scale: byte `opsel` of the lane's scale register applies to column i, k = 32 g .. 32 g + 31.
// With A dword t = word t of the lane's 16-byte unit (unit 4 ub + g of the row), nibble e at class p is bit
// 4 e + p of that word, i.e. column 32 t + elem(4 e + p) of the unit, elem(b) = b < 16 ? 2 (15 - b) :
// 2 (31 - b) + 1 (the "half2" order).  So B lane g needs, for class p, the 16 bytes (words 2 (g & 1),
// 2 (g & 1) + 1; e = 0..7) of unit 4 ub + (g >> 1) and the same of unit 4 ub + 2 + (g >> 1), and the scale of
// lane g is the one of unit 4 ub + g: the four bytes of a lane's scale register are the scales of its unit for
// class 0..3 (exponent + 2, + 1, + 0, + 0).
// LDS layout in 16-byte chunks: chunk(j, u, p, hf) = j * pitch + 8 u + 2 p + hf holds, for column j, unit u,
// class p, the bytes of words 2 hf, 2 hf + 1 (8 bytes each, e = 0..7).  pitch = 8 * units4 + 1 with units4 the
// number of staged units rounded up to a multiple of 4 (the padding is staged as zeros).  Scales: one dword per
// batch row and unit.
constexpr int kQ8Pieces = 3;
typedef int v8i_t __attribute__((ext_vector_type(8)));

__host__ __device__ constexpr int q8_units4(int units) { return (units + 3) & ~3; }
__host__ __device__ constexpr int q8_pitch(int units4) { return 8 * units4 + 1; }
__host__ __device__ constexpr int q8_chunks(int batch, int units4) { return batch * kQ8Pieces * q8_pitch(units4); }
// 16-byte chunks of unit scales (one dword per batch row and unit) in front of the pieces
__host__ __device__ constexpr int q8_scale_chunks(int batch, int units4) { return (batch * units4 + 3) / 4; }

template <int CTRL>
__device__ __forceinline__ uint32_t dpp_mov_u32(uint32_t v) {
    return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, CTRL, 0xF, 0xF, false);
}

// Lane q of a quad holds M_q (bytes c = 0..3); returns T with T byte e = byte q of M_{3-e}: a 4x4 byte
// transpose across the quad with the lane order reversed, two exchange-and-permute steps.
__device__ __forceinline__ uint32_t quad_transpose_rev(uint32_t m, bool odd, bool upper) {
    const uint32_t p1 = dpp_mov_u32<0xB1>(m);                       // lane ^ 1
    const uint32_t y = __builtin_amdgcn_perm(p1, m, odd ? 0x03070105u : 0x06020400u);
    const uint32_t p2 = dpp_mov_u32<0x4E>(y);                       // lane ^ 2
    return __builtin_amdgcn_perm(p2, y, upper ? 0x06070203u : 0x00010405u);
}

// Biased exponent eb of a unit's largest |u| (clamped so that an all-zero unit, an infinity or a NaN still give
// finite powers of two), the scale S = 2^(134 - eb) that brings it into [128, 256), its inverse, and the block
// scale bytes of the four classes: 2^(eb - 134) times 4, 2, 1, 1.
__device__ __forceinline__ uint32_t q8_exponent(uint32_t max_bits) { return min(max(max_bits >> 23, 32u), 240u); }
__device__ __forceinline__ float q8_scale(uint32_t eb) { return as_float((261u - eb) << 23); }
__device__ __forceinline__ float q8_inv_scale(uint32_t eb) { return as_float((eb - 7u) << 23); }
__device__ __forceinline__ uint32_t q8_scale_bytes(uint32_t eb) {
    const uint32_t e8 = eb - 7u;
    return (e8 + 2u) | ((e8 + 1u) << 8) | (e8 << 16) | (e8 << 24);
}

// Stage units [c0, c0 + cu_n) (plus zero padding up to q8_units4(cu_n)) of BATCH rows: pieces into xq, unit scales
// into scl[b * (pitch - 1) / 8 + unit], and xtot[b] (zeroed by the caller, barrier before) += the sum of the staged values in
// the columns of classes 0..2.  One pass, no barrier inside: a lane holds the 8 columns of one chunk, the 16 lanes
// of a DPP row hold one unit, so the unit maximum never leaves the row.  A barrier must follow before the staged
// data is read.
// DET (reproducible sums): xtot is [wavefronts][4] instead, every wavefront adds to its own entries (in program order,
// no atomics), and *ebmax (zeroed by the caller) receives the largest unit exponent eb of the staged chunk.
template <int DT, int BATCH, int THREADS, bool DET = false>
__device__ __forceinline__ void stage_units_q8(uint4* xq, uint32_t* scl, float* xtot, const StageInput& st, int c0,
                                               int cu_n, int pitch, uint32_t* ebmax = nullptr) {
    static_assert(!DET || BATCH <= 4, "per-wavefront totals are laid out [wavefront][4]");
    using E = Elem<DT>;
    constexpr int kBurst = 2;                            // chunks per lane in flight
    const int units4 = q8_units4(cu_n);
    const int nchunks = units4 * 16;                     // 8-column chunks per batch row, a multiple of 64
    const int total = BATCH * nchunks;
    const int lane = threadIdx.x & 63;
    const uint32_t esize = st.in_f32 ? 4u : 2u;
    const bool fast = st.vec_in && (st.K & 7) == 0;
    const __amdgpu_buffer_rsrc_t rin = raw_buffer(st.in, (uint32_t)(((size_t)(BATCH - 1) * st.in_stride + st.K) * esize));
    const bool scaled = !st.in_f32 && st.s_col != nullptr;
    const __amdgpu_buffer_rsrc_t rsc = raw_buffer(scaled ? (const void*)st.s_col : st.in, scaled ? (uint32_t)st.K * 2u : 0u);
    const bool coherent = st.in_f32 && st.in_coherent;
    const float rcp = 1.f / (float)nchunks;
    auto batch_row = [&](int it) -> int { return BATCH == 1 ? 0 : small_div(it, nchunks, rcp); };

    auto issue = [&](int it, u32x4_t& ra, u32x4_t& rb) {
        const int b = batch_row(it), q = it - b * nchunks;
        const int col = c0 * 128 + 8 * q;
        const bool live = fast && it < total && col < st.K;
        const uint32_t off = live ? (uint32_t)(((size_t)b * st.in_stride + col) * esize) : kPastEnd;
        if (coherent) {
            ra = __builtin_amdgcn_raw_buffer_load_b128(rin, off, 0, kCacheAgentCoherent);
            rb = __builtin_amdgcn_raw_buffer_load_b128(rin, live ? off + 16u : kPastEnd, 0, kCacheAgentCoherent);
        } else {
            ra = __builtin_amdgcn_raw_buffer_load_b128(rin, off, 0, kCacheDefault);
            if (st.in_f32) rb = __builtin_amdgcn_raw_buffer_load_b128(rin, live ? off + 16u : kPastEnd, 0, kCacheDefault);
            else rb = __builtin_amdgcn_raw_buffer_load_b128(rsc, live ? (uint32_t)col * 2u : kPastEnd, 0, kCacheDefault);
        }
    };
    // the 8 values of chunk (b, q) as fp32, input scale applied
    auto values = [&](int it, const u32x4_t& ra, const u32x4_t& rb, float (&v)[8]) {
        if (fast) {
            if (!st.in_f32) {
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const uint32_t xw = ra[e], sw = scaled ? rb[e] : E::kOnePair;
                    v[2 * e] = E::to_float(xw & 0xFFFFu) * E::to_float(sw & 0xFFFFu);
                    v[2 * e + 1] = E::to_float(xw >> 16) * E::to_float(sw >> 16);
                }
            } else {
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    v[e] = as_float(ra[e]);
                    v[4 + e] = as_float(rb[e]);
                }
            }
        } else {
            // element-wise fallback: odd K or rows that allow no 16-byte loads
            const int b = batch_row(it), q = it - b * nchunks;
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const int c = c0 * 128 + 8 * q + e;
                float t = 0.f;
                if (it < total && c < st.K) {
                    if (!st.in_f32) {
                        t = E::to_float(((const uint16_t*)st.in)[(size_t)b * st.in_stride + c]);
                        if (st.s_col) t *= E::to_float(st.s_col[c]);
                    } else if (st.in_coherent) {
                        t = __builtin_bit_cast(float, __hip_atomic_load((const uint32_t*)st.in + (size_t)b * st.in_stride + c,
                                                                        __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT));
                    } else {
                        t = ((const float*)st.in)[(size_t)b * st.in_stride + c];
                    }
                }
                v[e] = t;
            }
        }
    };
    // chunk (b, q): unit scale, pieces into LDS, and the chunk's share of xtot
    auto quantize = [&](int it, float (&v)[8]) -> float {
        const int b = batch_row(it), q = it - b * nchunks;
        const int cu = q >> 4, t = (q >> 2) & 3, qq = q & 3;
        float m = 0.f;
#pragma unroll
        for (int e = 0; e < 8; ++e) m = fmaxf(m, fabsf(v[e]));
        uint32_t mb = __builtin_bit_cast(uint32_t, m);
        mb = max(mb, dpp_mov_u32<0xB1>(mb));                // the 16 lanes of a DPP row hold one unit
        mb = max(mb, dpp_mov_u32<0x4E>(mb));
        mb = max(mb, dpp_mov_u32<0x141>(mb));
        mb = max(mb, dpp_mov_u32<0x140>(mb));
        const uint32_t eb = q8_exponent(mb);
        const float S = q8_scale(eb);
        float u[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) u[e] = v[e] * S;
        const float before = ((u[2] + u[3]) + (u[4] + u[5])) + (u[6] + u[7]);
        uint2* dst = (uint2*)xq + 2 * ((size_t)(b * kQ8Pieces) * pitch + 8 * cu + 2 * qq + (t >> 1)) + (t & 1);
#pragma unroll
        for (int k = 0; k < kQ8Pieces; ++k) {
            // class p = 0..3 <-> elements 6, 4, 2, 0 (even) and 7, 5, 3, 1 (odd) of the chunk
            int lo = __builtin_amdgcn_cvt_pk_fp8_f32(u[6], u[4], 0, false);
            lo = __builtin_amdgcn_cvt_pk_fp8_f32(u[2], u[0], lo, true);
            int hi = __builtin_amdgcn_cvt_pk_fp8_f32(u[7], u[5], 0, false);
            hi = __builtin_amdgcn_cvt_pk_fp8_f32(u[3], u[1], hi, true);
            {   // residuals: what the following pieces (or nobody) still have to carry
                const auto l0 = __builtin_amdgcn_cvt_pk_f32_fp8(lo, false), l1 = __builtin_amdgcn_cvt_pk_f32_fp8(lo, true);
                const auto h0 = __builtin_amdgcn_cvt_pk_f32_fp8(hi, false), h1 = __builtin_amdgcn_cvt_pk_f32_fp8(hi, true);
                u[6] -= l0[0]; u[4] -= l0[1]; u[2] -= l1[0]; u[0] -= l1[1];
                u[7] -= h0[0]; u[5] -= h0[1]; u[3] -= h1[0]; u[1] -= h1[1];
            }
            // classes 0..2 ride negated (bytes 0..2 of the packed quadruples)
            uint2 out;
            out.x = quad_transpose_rev((uint32_t)lo ^ 0x00808080u, lane & 1, lane & 2);
            out.y = quad_transpose_rev((uint32_t)hi ^ 0x00808080u, lane & 1, lane & 2);
            if (it < total) dst[(size_t)k * pitch * 2] = out;
        }
        if (it < total && (q & 15) == 0) {
            scl[b * ((pitch - 1) >> 3) + cu] = q8_scale_bytes(eb);
            if constexpr (DET) atomicMax(ebmax, eb);
        }
        // sum of the staged values (= input - last residual) over the columns of classes 0..2, in the input's units
        const float after = ((u[2] + u[3]) + (u[4] + u[5])) + (u[6] + u[7]);
        return (before - after) * q8_inv_scale(eb);
    };

#pragma unroll 1
    for (int it0 = threadIdx.x; it0 - lane < total; it0 += kBurst * THREADS) {     // wave-uniform trip count
        u32x4_t ra[kBurst], rb[kBurst];
#pragma unroll
        for (int j = 0; j < kBurst; ++j) issue(it0 + j * THREADS, ra[j], rb[j]);
        // A wavefront whose 64 chunks of a burst slot all lie past the end skips the slot's arithmetic (a short input
        // keeps only the first wavefronts busy, and the second slot is empty for every input of up to 8 x THREADS
        // columns per batch row): the branch is wave-uniform.
        const int wave_first = __builtin_amdgcn_readfirstlane(it0 - lane);
        float tot[kBurst];
#pragma unroll
        for (int j = 0; j < kBurst; ++j) {
            tot[j] = 0.f;
            if (wave_first + j * THREADS < total) {
                float v[8];
                values(it0 + j * THREADS, ra[j], rb[j], v);
                tot[j] = quantize(it0 + j * THREADS, v);
            }
        }
        // a wavefront's 64 chunks belong to one batch row (nchunks is a multiple of 64): one LDS atomic per
        // wavefront and burst slot
#pragma unroll
        for (int j = 0; j < kBurst; ++j) {
            const int it = it0 + j * THREADS;
            const float t = group_sum_tail(tot[j], 64);
            if (lane == 63 && it - lane < total) {
                if constexpr (DET) xtot[(threadIdx.x >> 6) * 4 + (it - lane) / nchunks] += t;
                else atomicAdd(&xtot[(it - lane) / nchunks], t);
            }
        }
    }
}

// One pass of a wavefront over a (row block, input chunk) of a stage whose words are in tile order: where its items
// lie and how many there are.  All members are wave-uniform.
struct Q8Pass {
    const uint32_t* bits;           // the stage's packed words
    uint32_t bytes;                 // their size
    int item_base;                  // item index of (first row pair, first unit group) of the pass; an item is the 2 KiB
                                    // at item index * 2048, the items of a row pair are consecutive
    int ngroups, skip;              // unit groups of the pass, and of the stage's rows outside the pass
    int it_begin, count;            // this wavefront's items: [it_begin, it_begin + count) of the pass, unit group fastest
};

// The B operand of one unit group held in registers: per class p the two 16-byte halves read from
// xq + column * pitch + 8 * (4 ub + (g >> 1)) + (g & 1) + 2 p (lo) and 16 chunks further (hi).  Named native
// vectors on purpose: arrays of uint4 captured by a lambda end up in scratch memory.
struct Q8Operand {
    u32x4_t lo0, lo1, lo2, lo3, hi0, hi1, hi2, hi3;
};

__device__ __forceinline__ void q8_read_operand(Q8Operand& o, const uint4* bp) {
    const u32x4_t* p = (const u32x4_t*)bp;
    o.lo0 = p[0]; o.hi0 = p[16];
    o.lo1 = p[2]; o.hi1 = p[18];
    o.lo2 = p[4]; o.hi2 = p[20];
    o.lo3 = p[6]; o.hi3 = p[22];
}

// One class of two row groups that share the input operand; `scale` holds the lane's four class scales, byte P is
// picked by the instruction.  All four classes add into ONE accumulator per row group; the two row groups
// alternate, which keeps dependent MFMAs two issues apart.
template <int P>
__device__ __forceinline__ void q8_class_pair(const uint4& wa, const uint4& wb, const u32x4_t& lo, const u32x4_t& hi,
                                              int scale, float4_t& acc_a, float4_t& acc_b) {
    constexpr uint32_t M = 0x11111111u << P;
    constexpr uint32_t C = P == 3 ? 0x22222222u : 0u;   // P == 3: the packed bit is the sign of 1.0
    constexpr int kOneScale = 0x7F7F7F7F;               // 2^0 for the weights
    const v8i_t b = {(int)lo.x, (int)lo.y, (int)lo.z, (int)lo.w, (int)hi.x, (int)hi.y, (int)hi.z, (int)hi.w};
    const v8i_t aa = {(int)((wa.x & M) | C), (int)((wa.y & M) | C), (int)((wa.z & M) | C), (int)((wa.w & M) | C), 0, 0, 0, 0};
    const v8i_t ab = {(int)((wb.x & M) | C), (int)((wb.y & M) | C), (int)((wb.z & M) | C), (int)((wb.w & M) | C), 0, 0, 0, 0};
    acc_a = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(aa, b, acc_a, 4 /* A: fp4 */, 0 /* B: fp8 */, 0, kOneScale, P, scale);
    acc_b = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(ab, b, acc_b, 4, 0, 0, kOneScale, P, scale);
}

// acc += the signed sum (less the staged total of classes 0..2) per (row, column) of the lane, for the units
// wa / wb of two row groups 16 rows apart
__device__ __forceinline__ void unit_mfma_q8_pair(const uint4& wa, const uint4& wb, const Q8Operand& o, int scale,
                                                  float4_t& acc_a, float4_t& acc_b) {
    q8_class_pair<0>(wa, wb, o.lo0, o.hi0, scale, acc_a, acc_b);
    q8_class_pair<1>(wa, wb, o.lo1, o.hi1, scale, acc_a, acc_b);
    q8_class_pair<2>(wa, wb, o.lo2, o.hi2, scale, acc_a, acc_b);
    q8_class_pair<3>(wa, wb, o.lo3, o.hi3, scale, acc_a, acc_b);
}

// v rounded to the grid 2^-23 of the binade of c (c = 1.5 * 2^k, |v| < 2^(k-1)): sums of such values that stay below
// 2^(k-1) are exact in fp32, so they do not depend on the order of the additions.
__device__ __forceinline__ float grid_round(float v, float c) {
    float t = v + c;
    asm volatile("" : "+v"(t));
    return t - c;
}

// Sum over the kQ8Pieces neighbouring columns of a batch row; valid in the lane of the last piece.
__device__ __forceinline__ float q8_piece_sum(float v) {
    static_assert(kQ8Pieces == 3, "two shifted adds");
    const int i = __builtin_bit_cast(int, v);
    const float s1 = __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, i, 0x111 /* row_shr:1 */, 0xF, 0xF, true));
    const float s2 = __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, i, 0x112 /* row_shr:2 */, 0xF, 0xF, true));
    return v + s1 + s2;
}

}  // namespace nq
