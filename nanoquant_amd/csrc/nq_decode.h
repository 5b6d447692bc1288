// Shared device code of the matmul-free decode stages: staging of the (scaled) input vector in LDS
// and the arithmetic of one 16-byte unit of packed signs (4 words = 128 columns of one row).
//
// LDS layout of the staged input (per batch row b): 16-byte chunk (b, i, cu) at
// xs[(b*16 + i)*upad + cu] holds the 8 consecutive columns 128*(c0+cu) + 8*i .. +7 as 16-bit values;
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

// Stage units [c0, c0+cu_n) for BATCH rows.  All threads of the workgroup call this; nthreads is the
// workgroup size (a multiple of 64).  Must be followed by a barrier before xs/xsum are read.
template <int DT, int BATCH>
__device__ __forceinline__ void stage_units(uint4* xs, float* xsum, const StageInput& st, int c0, int cu_n, int upad,
                                            int nthreads) {
    using E = Elem<DT>;
    if (st.in_f32 && st.in_coherent) {
        // Device-coherent loads are not served from this XCD's L2: keep them dense -- consecutive
        // lanes read consecutive pairs, one wavefront covers exactly one unit (64 pairs).
        const int npairs = cu_n * 64;
        const bool wide = (((uintptr_t)st.in | ((uintptr_t)st.in_stride * 4)) & 7u) == 0;
#pragma unroll 1
        for (int b = 0; b < BATCH; ++b) {
            const uint32_t* hp = (const uint32_t*)st.in + (size_t)b * st.in_stride;
            // kBurst loads per lane are put in flight before the first one is consumed: a coherent load is
            // a round trip to the memory side (~2 us); one round per burst instead of one per pair
            constexpr int kBurst = 4;
#pragma unroll 1
            for (int p0 = threadIdx.x; p0 < npairs; p0 += nthreads * kBurst) {
                uint32_t lo[kBurst], hi[kBurst];
#pragma unroll
                for (int j = 0; j < kBurst; ++j) {
                    const int p = p0 + j * nthreads;
                    const int col = c0 * 128 + 2 * p;
                    lo[j] = 0; hi[j] = 0;
                    if (p < npairs) {
                        if (wide && col + 1 < st.K) {
                            const uint64_t both = __hip_atomic_load((const uint64_t*)(hp + col), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                            lo[j] = (uint32_t)both; hi[j] = (uint32_t)(both >> 32);
                        } else {
                            if (col < st.K) lo[j] = __hip_atomic_load(hp + col, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                            if (col + 1 < st.K) hi[j] = __hip_atomic_load(hp + col + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                        }
                    }
                }
#pragma unroll
                for (int j = 0; j < kBurst; ++j) {
                    const int p = p0 + j * nthreads;
                    if (p < npairs) {      // wave-uniform: npairs and the wave's first p are multiples of 64
                        const uint16_t r0 = E::from_float(__builtin_bit_cast(float, lo[j]));
                        const uint16_t r1 = E::from_float(__builtin_bit_cast(float, hi[j]));
                        const int cu = p >> 6, i = (p & 63) >> 2, slot = p & 3;
                        ((uint32_t*)xs)[((b * 16 + i) * upad + cu) * 4 + slot] = (uint32_t)r0 | ((uint32_t)r1 << 16);
                        const float tot = group_sum(E::to_float(r0) + E::to_float(r1), 64);
                        if ((p & 63) == 0) xsum[b * upad + cu] = tot;
                    }
                }
            }
        }
        return;
    }
    const int nchunks = cu_n * 16;
    constexpr int kBurst = 2;   // chunks whose loads are in flight together
#pragma unroll 1
    for (int b = 0; b < BATCH; ++b) {
#pragma unroll 1
        for (int q0 = threadIdx.x; q0 < nchunks; q0 += nthreads * kBurst) {
            uint4 raw_a[kBurst], raw_b[kBurst];
            bool fast[kBurst];
#pragma unroll
            for (int j = 0; j < kBurst; ++j) {
                const int q = q0 + j * nthreads;
                const int col = (c0 + (q >> 4)) * 128 + (q & 15) * 8;
                fast[j] = q < nchunks && st.vec_in && col + 8 <= st.K;
                raw_a[j] = make_uint4(0, 0, 0, 0);
                raw_b[j] = make_uint4(E::kOnePair, E::kOnePair, E::kOnePair, E::kOnePair);
                if (fast[j]) {
                    if (!st.in_f32) {
                        raw_a[j] = *(const uint4*)((const uint16_t*)st.in + (size_t)b * st.in_stride + col);
                        if (st.s_col) raw_b[j] = *(const uint4*)(st.s_col + col);
                    } else {
                        const float* hp = (const float*)st.in + (size_t)b * st.in_stride + col;
                        raw_a[j] = *(const uint4*)hp;
                        raw_b[j] = *(const uint4*)(hp + 4);
                    }
                }
            }
#pragma unroll
            for (int j = 0; j < kBurst; ++j) {
                const int q = q0 + j * nthreads;
                if (q >= nchunks) continue;               // uniform over each aligned group of 16 lanes
                const int cu = q >> 4, i = q & 15;
                const int col = (c0 + cu) * 128 + i * 8;
                float v[8];
                if (fast[j]) {
                    if (!st.in_f32) {
#pragma unroll
                        for (int e = 0; e < 4; ++e) {
                            const uint32_t xw = comp_d(raw_a[j], e), sw = comp_d(raw_b[j], e);
                            v[2 * e] = E::to_float(xw & 0xFFFFu) * E::to_float(sw & 0xFFFFu);
                            v[2 * e + 1] = E::to_float(xw >> 16) * E::to_float(sw >> 16);
                        }
                    } else {
#pragma unroll
                        for (int e = 0; e < 4; ++e) {
                            v[e] = __builtin_bit_cast(float, comp_d(raw_a[j], e));
                            v[4 + e] = __builtin_bit_cast(float, comp_d(raw_b[j], e));
                        }
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
                uint16_t r[8];
                float tot = 0.f;
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    r[e] = E::from_float(v[e]);
                    tot += E::to_float(r[e]);          // the sum of what the dot products will actually see
                }
                uint4 p;
                p.x = (uint32_t)r[0] | ((uint32_t)r[1] << 16);
                p.y = (uint32_t)r[2] | ((uint32_t)r[3] << 16);
                p.z = (uint32_t)r[4] | ((uint32_t)r[5] << 16);
                p.w = (uint32_t)r[6] | ((uint32_t)r[7] << 16);
                xs[(b * 16 + i) * upad + cu] = p;
                // the 16 chunks of a unit are held by 16 consecutive lanes: finish the unit sum with DPP
                tot = group_sum(tot, 16);
                if (i == 0) xsum[b * upad + cu] = tot;
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
                const uint4 x0 = xs[(b * 16 + 4 * wi + 0) * upad + cu];
                const uint4 x1 = xs[(b * 16 + 4 * wi + 1) * upad + cu];
                const uint4 x2 = xs[(b * 16 + 4 * wi + 2) * upad + cu];
                const uint4 x3 = xs[(b * 16 + 4 * wi + 3) * upad + cu];
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
                for (int q = 0; q < 4; ++q) xv[q] = xs[(b * 16 + 4 * wi + q) * upad + cu];
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

// sign bits of `shifted` (bits 15 and 31) onto the pair (1.0, 1.0): one v_bfi_b32
__device__ __forceinline__ uint32_t sign_onto_one(uint32_t shifted, uint32_t one_pair) {
    uint32_t r;
    asm("v_bfi_b32 %0, %1, %2, %3" : "=v"(r) : "s"(kSignPair), "v"(shifted), "v"(one_pair));
    return r;
}

// acc += signs(w: this lane's unit) x staged activations of unit `cu` (zero contribution when !valid).
// xs row used by this lane: batch row min(lane & 15, BATCH-1); columns beyond BATCH are never read back.
template <int DT, int BATCH>
__device__ __forceinline__ void unit_mfma(const uint4& w, const uint4* xs, int upad, int cu, bool valid, float4_t& acc) {
    using E = Elem<DT>;
    const int nb = min((int)(threadIdx.x & 15), BATCH - 1);
    const uint32_t one = E::kOnePair;
#pragma unroll
    for (int wi = 0; wi < 4; ++wi) {
        const uint32_t word = comp_d(w, wi);
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            uint4 a;
            a.x = sign_onto_one(word << (4 * q + 0), one);
            a.y = sign_onto_one(word << (4 * q + 1), one);
            a.z = sign_onto_one(word << (4 * q + 2), one);
            a.w = sign_onto_one(word << (4 * q + 3), one);
            uint4 b = make_uint4(0, 0, 0, 0);
            if (valid) b = xs[(nb * 16 + 4 * wi + q) * upad + cu];
            acc = Mfma16<DT>::run(a, b, acc);
        }
    }
}

}  // namespace nq
