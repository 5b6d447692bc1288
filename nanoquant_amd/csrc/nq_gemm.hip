// Prefill path (>= 128 tokens): one-bit weights x 16-bit activations on the MFMA units of gfx950.
//
//   C[t, j] = s_out[j] * sum_k (x[t, k] * s_in[k]) * sgn(W[j, k])
//
// Replaces Marlin_impl / marlin_cuda_template of the reference (src/nanoquant/kernel/cuda/
// gemm_kernel.cu:278-932) in function only.  Design for CDNA4: the sign words never touch LDS.  The
// weight matrix is stored in 1 KiB tiles of 32 rows x 256 k (packing.py: pack_gemm_tiles) so that a
// wavefront fetches one tile with a single 128-bit load per lane and expands it in registers: the
// 8 k-values a lane feeds to v_mfma_f32_32x32x16 are one byte of its 16, and `(word << s) &
// 0x80008000 | (1.0, 1.0)` turns two of those bits into a +-1 pair, so the B operand is built with
// integer logic only.  Activations (scaled by s_in while staging) are the A operand and come from an
// LDS slab shared by the four wavefronts of a workgroup; accumulation is fp32 in the MFMA
// accumulators.  With A = activations the result registers of a lane run along the output row index,
// which makes the epilogue stores contiguous.
//
// Work split: grid.x = 128-row blocks (4 wavefronts x 32 rows), grid.y = token blocks of 32*TT,
// grid.z = k-splits.  With one k-split the epilogue scales and stores directly; otherwise partial
// sums are added into an fp32 scratch with hardware float atomics and a small second kernel scales
// and converts (and re-zeroes the scratch, which must be zero on entry).
#include "nq_common.h"
#include "nq_kernels.h"

namespace nq {

struct GemmArgs {
    const void* x;          // [T, K] 16-bit
    const uint4* tiles;     // [R/32][K/256][64 lanes] 16 bytes each
    const uint16_t* s_in;   // [K] or null
    const uint16_t* s_out;  // [R] or null
    void* y;                // [T, R] 16-bit
    float* acc;             // [T, R] fp32 partial sums (k-split only)
    int T, K, R;
    int ktiles;             // K / 256
    int ktiles_per_split;
};

constexpr int kSlabK = 256;
constexpr int kPitch = kSlabK + 8;  // 16-bit elements per LDS row: 528 bytes, conflict-free b128 reads

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

template <int DT, int TT, bool SPLIT>
__global__ __launch_bounds__(256) void gemm_onebit_kernel(GemmArgs a) {
    using E = Elem<DT>;
    extern __shared__ uint16_t slab[];  // [32*TT][kPitch]
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int rt = blockIdx.x * 4 + wave;          // 32-row tile of this wavefront
    const bool have_rows = rt * 32 < a.R;
    const int tok0 = blockIdx.y * (32 * TT);
    const int kt_begin = blockIdx.z * a.ktiles_per_split;
    const int kt_end = min(kt_begin + a.ktiles_per_split, a.ktiles);

    float16_t acc[TT];
#pragma unroll
    for (int tt = 0; tt < TT; ++tt)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[tt][v] = 0.f;

    const uint4* tile_ptr = a.tiles + ((size_t)rt * a.ktiles + kt_begin) * 64 + lane;
    uint4 wnext = make_uint4(0, 0, 0, 0);
    if (have_rows && kt_begin < kt_end) wnext = *tile_ptr;

#pragma unroll 1
    for (int kt = kt_begin; kt < kt_end; ++kt) {
        // ---- stage the activation slab [32*TT tokens][256 k], scaled by s_in, zero beyond T ----
        if (kt != kt_begin) __syncthreads();
        const int k0 = kt * kSlabK;
#pragma unroll
        for (int pass = 0; pass < TT * 4; ++pass) {
            const int q = pass * 256 + threadIdx.x;   // 16-byte chunk id: 32 chunks per token row
            const int trow = q >> 5, c8 = (q & 31) * 8;
            const int tok = tok0 + trow;
            uint4 xv = make_uint4(0, 0, 0, 0);
            if (tok < a.T) {
                xv = *(const uint4*)((const uint16_t*)a.x + (size_t)tok * a.K + k0 + c8);
                if (a.s_in) {
                    const uint4 sv = *(const uint4*)(a.s_in + k0 + c8);
                    uint32_t o[4];
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const uint32_t xw = comp4(xv, e), sw = comp4(sv, e);
                        const float lo = E::to_float(xw & 0xFFFFu) * E::to_float(sw & 0xFFFFu);
                        const float hi = E::to_float(xw >> 16) * E::to_float(sw >> 16);
                        o[e] = (uint32_t)E::from_float(lo) | ((uint32_t)E::from_float(hi) << 16);
                    }
                    xv = make_uint4(o[0], o[1], o[2], o[3]);
                }
            }
            *(uint4*)(slab + trow * kPitch + c8) = xv;
        }
        const uint4 w = wnext;
        if (have_rows && kt + 1 < kt_end) wnext = tile_ptr[(size_t)(kt + 1 - kt_begin) * 64];
        __syncthreads();

        if (have_rows) {
#pragma unroll
            for (int t = 0; t < 16; ++t) {
                const uint32_t word = comp4(w, t >> 2);
                const int s = 4 * (t & 3);
                uint4 bfrag;
                bfrag.x = ((word << (s + 0)) & kSignPair) | E::kOnePair;
                bfrag.y = ((word << (s + 1)) & kSignPair) | E::kOnePair;
                bfrag.z = ((word << (s + 2)) & kSignPair) | E::kOnePair;
                bfrag.w = ((word << (s + 3)) & kSignPair) | E::kOnePair;
#pragma unroll
                for (int tt = 0; tt < TT; ++tt) {
                    const uint4 afrag = *(const uint4*)(slab + (tt * 32 + (lane & 31)) * kPitch + 16 * t + 8 * (lane >> 5));
                    acc[tt] = Mfma<DT>::run(afrag, bfrag, acc[tt]);
                }
            }
        }
    }

    if (!have_rows) return;
    const int row = rt * 32 + (lane & 31);
    float sc = 1.f;
    if (!SPLIT && a.s_out) sc = E::to_float(a.s_out[row]);
#pragma unroll
    for (int tt = 0; tt < TT; ++tt) {
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            const int tok = tok0 + tt * 32 + 8 * (v >> 2) + 4 * (lane >> 5) + (v & 3);
            if (tok < a.T) {
                const size_t o = (size_t)tok * a.R + row;
                if (SPLIT) atomicAdd(a.acc + o, acc[tt][v]);
                else ((uint16_t*)a.y)[o] = E::from_float_sat(acc[tt][v] * sc);
            }
        }
    }
}

// Scales, converts and stores the accumulated sums, and puts the accumulator back to zero: the scratch
// is zero on entry of every GEMM call and zero again when the call has finished.
template <int DT>
__global__ __launch_bounds__(256) void gemm_finish_kernel(float4* acc, const uint16_t* s_out, uint16_t* y, int R, size_t n4) {
    using E = Elem<DT>;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n4; i += stride) {
        const float4 v = acc[i];
        acc[i] = make_float4(0.f, 0.f, 0.f, 0.f);
        const int row = (int)((i * 4) % (size_t)R);   // R % 4 == 0, so the 4 values share a token
        float s0 = 1.f, s1 = 1.f, s2 = 1.f, s3 = 1.f;
        if (s_out) {
            s0 = E::to_float(s_out[row]); s1 = E::to_float(s_out[row + 1]);
            s2 = E::to_float(s_out[row + 2]); s3 = E::to_float(s_out[row + 3]);
        }
        uint2 o;
        o.x = (uint32_t)E::from_float_sat(v.x * s0) | ((uint32_t)E::from_float_sat(v.y * s1) << 16);
        o.y = (uint32_t)E::from_float_sat(v.z * s2) | ((uint32_t)E::from_float_sat(v.w * s3) << 16);
        ((uint2*)y)[i] = o;
    }
}

// ---- host side --------------------------------------------------------------------------------
struct GemmPlan {
    int tt;       // 32-token tiles per wavefront
    int gx, gy, ksplit, ktiles_per_split;
};

static GemmPlan plan_gemm(int T, int K, int R) {
    GemmPlan p;
    // 64-token blocks measured faster than 128-token blocks at 128 and 512 tokens alike: twice the
    // workgroups, half the slab to stage between barriers.
    p.tt = 2;
    p.gx = (R + 127) / 128;
    p.gy = (T + 32 * p.tt - 1) / (32 * p.tt);
    const int ktiles = K / kSlabK;
    int want = 512 / (p.gx * p.gy);          // k-splits needed to put two workgroups on every CU
    if (want < 1) want = 1;
    int max_split = ktiles / 2;              // keep at least 512 k per split
    if (max_split < 1) max_split = 1;
    int ks = want < max_split ? want : max_split;
    p.ktiles_per_split = (ktiles + ks - 1) / ks;
    p.ksplit = (ktiles + p.ktiles_per_split - 1) / p.ktiles_per_split;
    return p;
}

size_t gemm_scratch_bytes(int T, int K, int R) {
    if (T <= 0 || K <= 0 || R <= 0 || K % kSlabK != 0) return 0;
    const GemmPlan p = plan_gemm(T, K, R);
    return p.ksplit > 1 ? (size_t)T * R * sizeof(float) : 0;
}

template <int DT, int TT>
static hipError_t launch_gemm(const GemmArgs& a, const GemmPlan& p, hipStream_t stream) {
    const size_t lds = (size_t)32 * TT * kPitch * sizeof(uint16_t);
    dim3 grid(p.gx, p.gy, p.ksplit);
    if (p.ksplit > 1) {
        auto kern = gemm_onebit_kernel<DT, TT, true>;
        static bool attr_done = false;
        if (lds > 64 * 1024 && !attr_done) {
            hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
            if (e != hipSuccess) return e;
            attr_done = true;
        }
        const size_t n4 = (size_t)a.T * a.R / 4;
        size_t zb = (n4 + 255) / 256;
        if (zb > 2048) zb = 2048;
        hipLaunchKernelGGL(kern, grid, dim3(256), lds, stream, a);
        hipLaunchKernelGGL(gemm_finish_kernel<DT>, dim3((unsigned)zb), dim3(256), 0, stream, (float4*)a.acc, a.s_out,
                           (uint16_t*)a.y, a.R, n4);
    } else {
        auto kern = gemm_onebit_kernel<DT, TT, false>;
        static bool attr_done = false;
        if (lds > 64 * 1024 && !attr_done) {
            hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
            if (e != hipSuccess) return e;
            attr_done = true;
        }
        hipLaunchKernelGGL(kern, grid, dim3(256), lds, stream, a);
    }
    return hipGetLastError();
}

// Shapes must satisfy K % 256 == 0 and R % 32 == 0 (checked by the caller).  `scratch` (when
// gemm_scratch_bytes > 0) must be zero on entry and is zero again when the enqueued work has finished.
hipError_t gemm_onebit(int dtype, const void* x, const uint32_t* tiles, const void* s_in, const void* s_out,
                       void* y, float* scratch, int T, int K, int R, hipStream_t stream) {
    GemmArgs a;
    a.x = x; a.tiles = (const uint4*)tiles;
    a.s_in = (const uint16_t*)s_in; a.s_out = (const uint16_t*)s_out;
    a.y = y; a.acc = scratch;
    a.T = T; a.K = K; a.R = R;
    a.ktiles = K / kSlabK;
    const GemmPlan p = plan_gemm(T, K, R);
    a.ktiles_per_split = p.ktiles_per_split;
    if (dtype == 0) return p.tt == 2 ? launch_gemm<0, 2>(a, p, stream) : launch_gemm<0, 4>(a, p, stream);
    return p.tt == 2 ? launch_gemm<1, 2>(a, p, stream) : launch_gemm<1, 4>(a, p, stream);
}

}  // namespace nq
