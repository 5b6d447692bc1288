// Decode path (batch 1..16): matmul-free binary GEMV stages for gfx950.
//
// One stage computes, for a packed sign matrix W [rows, words] in the row-major "half2" word order,
//     out[b, row] = s_row[row] * sum_c sgn(W[row, c]) * (in[b, c] * s_col[c])
// A layer is two stages: rows = rank over K = in_features (input x, scales s_in / s_mid, fp32 result h),
// then rows = out_features over K = rank (input h, scale s_out, result y in the activation type).
// Replaces nanoquant_stage1_impl / nanoquant_stage2_impl of the reference
// (src/nanoquant/kernel/cuda/gemv_kernel.cu:43-277), with three differences that are the point of
// the design: every packed word is fetched once for all batch rows (the reference re-reads the
// weights per batch row, :288-290), the sign words arrive as 128-bit loads with no intra-quad
// redundancy (:93), and all sums are carried in fp32 (the reference sums in fp16, :103-106).
//
// Mapping: a workgroup of 4 wavefronts stages the scaled input vector(s) once in LDS as 16-bit pairs.
// A wavefront is split into 64/G lane groups; a lane group owns RPW rows and its G lanes stride over
// the row's 16-byte units (4 words = 128 columns).  The arithmetic of a unit (masked words used
// directly as the second operand of v_dot2_f32_{f16,bf16}, fp32 accumulators) is in nq_decode.h.
// Row sums are finished with DPP moves inside a 16-lane row and two ds_bpermute steps.
#include "nq_decode.h"
#include "nq_kernels.h"

namespace nq {

struct StageArgs {
    const uint32_t* bits;   // [rows, words]
    const void* in;         // [batch, in_stride]: 16-bit activations (FIRST) or fp32 h (!FIRST)
    const uint16_t* s_col;  // [K] per-column scale (FIRST only), may be null
    const uint16_t* s_row;  // [rows] per-row scale, may be null
    void* out;              // [batch, out_stride]: fp32 h (FIRST) or 16-bit y (!FIRST)
    int rows, words, K;     // K = logical columns, K <= 32*words
    int in_stride, out_stride;
    int group_log2;         // lanes per row = 1 << group_log2
    int units;              // 16-byte units per row = ceil(words / 4)
    int chunk_units;        // units staged in LDS per pass
    int vec_bits;           // rows of `bits` are 16-byte aligned and words % 4 == 0
    int vec_in;             // rows of `in` (and s_col) allow 16-byte loads
    const float* addend;    // [batch, out_stride] fp32 added before the store (sum over terms), may be null
    const uint16_t* bias;   // [rows] added after the row scale, may be null
    int out_f32;            // store fp32 instead of the 16-bit activation type
};

template <int RPW>
__device__ __forceinline__ void load_bits(uint4 (&w)[RPW], const StageArgs& a, int row0, int unit, bool active) {
#pragma unroll
    for (int rr = 0; rr < RPW; ++rr) {
        w[rr] = make_uint4(0, 0, 0, 0);
        if (!active) continue;
        const int row = min(row0 + rr, a.rows - 1);
        const uint32_t* p = a.bits + (size_t)row * a.words + 4 * unit;
        if (a.vec_bits) {
            typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
            const u32x4 v = __builtin_nontemporal_load((const u32x4*)p);
            w[rr] = make_uint4(v.x, v.y, v.z, v.w);
        } else {
            const int left = a.words - 4 * unit;
            w[rr].x = p[0];
            if (left > 1) w[rr].y = p[1];
            if (left > 2) w[rr].z = p[2];
            if (left > 3) w[rr].w = p[3];
        }
    }
}

template <int DT, bool FIRST, int BATCH, int RPW>
__global__ __launch_bounds__(256) void gemv_stage_kernel(StageArgs a) {
    using E = Elem<DT>;
    extern __shared__ uint4 lds_raw[];
    float* xsum = (float*)lds_raw;                       // [BATCH][kXsumStride] per-unit input sums
    uint4* lds = lds_raw + (BATCH * kXsumStride * sizeof(float)) / sizeof(uint4);
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    StageInput sin;
    sin.in = a.in; sin.s_col = a.s_col; sin.K = a.K; sin.in_stride = a.in_stride;
    sin.in_f32 = FIRST ? 0 : 1; sin.in_coherent = 0; sin.vec_in = a.vec_in;
    const int G = 1 << a.group_log2;
    const int g = lane & (G - 1), slot = lane >> a.group_log2;
    const int rows_per_wave = (kWave >> a.group_log2) * RPW;
    const int row0 = (blockIdx.x * (blockDim.x >> 6) + wave) * rows_per_wave + slot * RPW;
    const int upad = a.chunk_units | 1;

    float acc[RPW][BATCH];
#pragma unroll
    for (int rr = 0; rr < RPW; ++rr)
#pragma unroll
        for (int b = 0; b < BATCH; ++b) acc[rr][b] = 0.f;

    // The sign words do not depend on the activations: put the first fetch in flight before staging.
    uint4 wnext[RPW];
    load_bits<RPW>(wnext, a, row0, g, g < min(a.chunk_units, a.units) && row0 < a.rows);

#pragma unroll 1
    for (int c0 = 0; c0 < a.units; c0 += a.chunk_units) {
        const int cu_n = min(a.chunk_units, a.units - c0);
        if (c0) __syncthreads();
        stage_units<DT, BATCH>(lds, xsum, sin, c0, cu_n, upad, (int)blockDim.x);
        __syncthreads();
#pragma unroll 1
        for (int cu = g; cu - g < cu_n; cu += G) {
            uint4 w[RPW];
#pragma unroll
            for (int rr = 0; rr < RPW; ++rr) w[rr] = wnext[rr];
            const bool active = cu < cu_n && row0 < a.rows;
            {   // next fetch: same chunk, or the first iteration of the following chunk
                int ncu = cu + G, nc0 = c0;
                if (ncu - g >= cu_n) { nc0 = c0 + a.chunk_units; ncu = g; }
                const bool nact = nc0 < a.units && ncu < min(a.chunk_units, a.units - nc0) && row0 < a.rows;
                load_bits<RPW>(wnext, a, row0, nc0 + ncu, nact);
            }
            if (active) {
#pragma unroll
                for (int rr = 0; rr < RPW; ++rr) {
                    float part[BATCH];
                    UnitDot<DT, BATCH>::run(w[rr], lds, xsum, upad, cu, part);
#pragma unroll
                    for (int b = 0; b < BATCH; ++b) acc[rr][b] += part[b];
                }
            }
        }
    }

#pragma unroll
    for (int rr = 0; rr < RPW; ++rr) {
        const int row = row0 + rr;
        float sc = 1.f, bs = 0.f;
        if (a.s_row && row < a.rows) sc = E::to_float(a.s_row[row]);
        if (a.bias && row < a.rows) bs = E::to_float(a.bias[row]);
#pragma unroll
        for (int b = 0; b < BATCH; ++b) {
            float v = group_sum(acc[rr][b], G) * sc + bs;
            if (g == 0 && row < a.rows) {
                const size_t o = (size_t)b * a.out_stride + row;
                if (a.addend) v += a.addend[o];
                if (a.out_f32) ((float*)a.out)[o] = v;
                else ((uint16_t*)a.out)[o] = E::from_float_clamped(v);
            }
        }
    }
}

// ---- host side --------------------------------------------------------------------------------
static int pick_group_log2(int units, int rows, int batch) {
    if (batch == 1) {
        // One batch row is bound by how many bytes are in flight: a small lane group puts many rows into a workgroup
        // and leaves few workgroups (rank 3008 x 11008 columns: 86 units, 8 lanes per row, 94 workgroups on 256 CUs,
        // 14 us).  Take the lane group that maximises (share of lanes on real data) x (workgroups, up to what the
        // device keeps resident), the smaller group on ties (Llama-2-7B layer: 80 -> 74 us; with more batch rows the
        // arithmetic per workgroup weighs more and the rule below stays faster).
        int best = 0;
        double best_score = -1.0;
        for (int gl = 0; gl <= 6; ++gl) {
            const int G = 1 << gl;
            const int passes = (units + G - 1) / G;
            double grid = (double)rows / (4 * (kWave / G));
            if (grid > 1536.0) grid = 1536.0;
            const double score = (double)units / (double)(G * passes) * grid;
            if (score > best_score * 1.001) { best_score = score; best = gl; }
        }
        return best;
    }
    // Largest lane group whose last pass still keeps >= 90% of the lanes on real data.
    int best = 0;
    for (int gl = 6; gl >= 0; --gl) {
        const int G = 1 << gl;
        const int passes = (units + G - 1) / G;
        if ((double)units / (double)(G * passes) >= 0.90) { best = gl; break; }
    }
    return best;
}

constexpr int kLdsBudget = 144 * 1024;
constexpr int kXsumBytesPerRow = kXsumStride * (int)sizeof(float);

template <int DT, bool FIRST, int BATCH, int RPW>
static hipError_t launch_stage(StageArgs a, hipStream_t stream) {
    const int rows_per_block = 4 * (kWave >> a.group_log2) * RPW;
    const int grid = (a.rows + rows_per_block - 1) / rows_per_block;
    const size_t lds_bytes = (size_t)BATCH * kXsumBytesPerRow + (size_t)xs_chunks(BATCH, a.chunk_units | 1) * sizeof(uint4);
    auto kern = gemv_stage_kernel<DT, FIRST, BATCH, RPW>;
    static PerDeviceFlag attr_done;  // per template instance and device; raised once to the full budget
    const int dev = current_device();
    if (lds_bytes > 64 * 1024 && !attr_done.test(dev)) {
        hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, kLdsBudget);
        if (e != hipSuccess) return e;
        attr_done.set(dev);
    }
    hipLaunchKernelGGL(kern, dim3(grid), dim3(256), lds_bytes, stream, a);
    return hipGetLastError();
}

template <int DT, bool FIRST, int BATCH>
static hipError_t launch_stage_rpw(StageArgs a, hipStream_t stream) {
    const int slots = kWave >> a.group_log2;
    // Two rows per lane group halve the LDS reads per sign bit; only when the grid still covers the chip.
    if (BATCH <= 4 && a.rows / (4 * slots * 2) >= 512) return launch_stage<DT, FIRST, BATCH, 2>(a, stream);
    return launch_stage<DT, FIRST, BATCH, 1>(a, stream);
}

template <int DT, bool FIRST>
static hipError_t launch_stage_batch(StageArgs a, int batch, hipStream_t stream) {
    switch (batch) {
        case 1: return launch_stage_rpw<DT, FIRST, 1>(a, stream);
        case 2: return launch_stage_rpw<DT, FIRST, 2>(a, stream);
        case 4: return launch_stage_rpw<DT, FIRST, 4>(a, stream);
        case 8: return launch_stage_rpw<DT, FIRST, 8>(a, stream);
        case 16: return launch_stage_rpw<DT, FIRST, 16>(a, stream);
        default: return hipErrorInvalidValue;
    }
}

static inline bool aligned16(const void* p) { return ((uintptr_t)p & 15u) == 0; }

// Pieces of 8 and 16 batch rows go through the run-list kernel on this one stage (MFMA unit arithmetic, us per
// Llama-2-7B layer: batch 8 157 vs 240, batch 16 225 vs 570); smaller pieces are as fast or faster on the lane-group
// kernel below, whose launches carry less fixed cost (batch 4: 131 vs 133, batch 1: 80 vs 111).
static bool use_stream_kernel(int piece) { return piece >= 8; }

// One stage over `batch` input rows, any batch >= 1: split into power-of-two pieces of at most 16.
hipError_t gemv_stage(int dtype, bool first, const uint32_t* bits, const void* in, const void* s_col,
                      const void* s_row, const float* addend, void* out, bool out_f32, int batch, int rows,
                      int words, int K, int in_stride, int out_stride, hipStream_t stream, const void* bias) {
    if (rows <= 0 || batch <= 0) return hipSuccess;
    StageArgs a;
    a.bits = bits;
    a.bias = (const uint16_t*)bias;
    a.s_col = (const uint16_t*)s_col;
    a.s_row = (const uint16_t*)s_row;
    a.rows = rows; a.words = words; a.K = K;
    a.in_stride = in_stride; a.out_stride = out_stride;
    a.units = (words + 3) / 4;
    a.vec_bits = (words % 4 == 0) && aligned16(bits);
    const size_t in_elt = first ? 2 : 4;
    a.vec_in = aligned16(in) && ((size_t)in_stride * in_elt) % 16 == 0 && (!s_col || aligned16(s_col));

    int done = 0;
    while (done < batch) {
        int piece = 16;
        while (piece > batch - done) piece >>= 1;
        int cap = (kLdsBudget - piece * kXsumBytesPerRow - piece * (int)sizeof(uint4)) / (piece * 16 * (int)sizeof(uint4));   // chunk_units|1 must fit
        cap = (cap - 1) & ~1;                                       // even, so that cap|1 <= budget
        if (cap > kXsumStride - 2) cap = kXsumStride - 2;
        a.chunk_units = a.units < cap ? a.units : cap;
        a.group_log2 = pick_group_log2(a.chunk_units, rows, piece);
        a.in = (const char*)in + (size_t)done * in_stride * in_elt;
        a.out = (char*)out + (size_t)done * out_stride * (out_f32 ? 4 : 2);
        a.addend = addend ? addend + (size_t)done * out_stride : nullptr;
        a.out_f32 = out_f32 ? 1 : 0;
        hipError_t e;
        if (use_stream_kernel(piece) && (size_t)rows * words * 4 < 0x7FFFFFF0ull) {
            RunStage st{};
            st.bits = bits; st.in = a.in; st.s_col = a.s_col; st.s_row = a.s_row; st.out = a.out; st.addend = a.addend; st.bias = a.bias;
            st.rows = rows; st.words = words; st.K = K; st.units = a.units;
            st.in_stride = in_stride; st.out_stride = out_stride;
            st.in_f32 = first ? 0 : 1; st.out_f32 = a.out_f32;
            st.dep = -1; st.dep2 = -1; st.signal = 0;
            st.vec_bits = a.vec_bits; st.vec_in = a.vec_in;
            st.phase = 0; st.seg_count = 0; st.in_coherent = 0; st.heavy_release = 0; st.heavy_acquire = 0;
            e = gemv_stream_single(dtype, piece, st, stream);
        } else if (dtype == 0) e = first ? launch_stage_batch<0, true>(a, piece, stream) : launch_stage_batch<0, false>(a, piece, stream);
        else e = first ? launch_stage_batch<1, true>(a, piece, stream) : launch_stage_batch<1, false>(a, piece, stream);
        if (e != hipSuccess) return e;
        done += piece;
    }
    return hipSuccess;
}

}  // namespace nq
