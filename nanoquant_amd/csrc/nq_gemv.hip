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

#include <atomic>

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

// What a second-stage workgroup of a fused launch waits for before it reads its input: `counter` reaching `target`
// (the number of first-stage workgroups of its linear), at most `spin_limit` polls.
struct StageWait {
    const unsigned* counter;
    unsigned target, spin_limit;
    unsigned* status;
};

// FUSED: both stages of a linear run in one launch.  The first stage stores h with device-coherent stores (another
// workgroup of the same launch reads it), the second stage waits (after its first fetch of sign words is in flight)
// until every first-stage workgroup of its linear has arrived, and stages h with device-coherent loads.
template <int DT, bool FIRST, int BATCH, int RPW, bool FUSED>
__device__ __forceinline__ void stage_body(const StageArgs& a, int block, const StageWait& wait) {
    using E = Elem<DT>;
    extern __shared__ uint4 lds_raw[];
    float* xsum = (float*)lds_raw;                       // [BATCH][kXsumStride] per-unit input sums
    uint4* lds = lds_raw + (BATCH * kXsumStride * sizeof(float)) / sizeof(uint4);
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    StageInput sin;
    sin.in = a.in; sin.s_col = a.s_col; sin.K = a.K; sin.in_stride = a.in_stride;
    sin.in_f32 = FIRST ? 0 : 1; sin.in_coherent = (FUSED && !FIRST) ? 1 : 0; sin.vec_in = a.vec_in;
    const int G = 1 << a.group_log2;
    const int g = lane & (G - 1), slot = lane >> a.group_log2;
    const int rows_per_wave = (kWave >> a.group_log2) * RPW;
    const int row0 = (block * (blockDim.x >> 6) + wave) * rows_per_wave + slot * RPW;
    const int upad = a.chunk_units | 1;

    float acc[RPW][BATCH];
#pragma unroll
    for (int rr = 0; rr < RPW; ++rr)
#pragma unroll
        for (int b = 0; b < BATCH; ++b) acc[rr][b] = 0.f;

    // The sign words do not depend on the activations: put the first fetch in flight before staging.
    uint4 wnext[RPW];
    load_bits<RPW>(wnext, a, row0, g, g < min(a.chunk_units, a.units) && row0 < a.rows);

    if constexpr (FUSED && !FIRST) {
        if (threadIdx.x == 0) {
            unsigned spins = 0;
            while (__hip_atomic_load(wait.counter, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) < wait.target) {
                __builtin_amdgcn_s_sleep(4);
                if (++spins >= wait.spin_limit) {            // bounded: report and go on (the outputs are then invalid)
                    atomicOr(wait.status, 1u);
                    break;
                }
            }
        }
        __syncthreads();
    }

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
                if (a.out_f32) {
                    if constexpr (FUSED && FIRST)
                        __hip_atomic_store((uint32_t*)a.out + o, __builtin_bit_cast(uint32_t, v), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    else
                        ((float*)a.out)[o] = v;
                } else {
                    ((uint16_t*)a.out)[o] = E::from_float_clamped(v);
                }
            }
        }
    }
}

template <int DT, bool FIRST, int BATCH, int RPW>
__global__ __launch_bounds__(256) void gemv_stage_kernel(StageArgs a) {
    stage_body<DT, FIRST, BATCH, RPW, false>(a, (int)blockIdx.x, StageWait{});
}

// Both stages of up to kFusedMax linears in ONE ordinary launch (no resident-grid requirement): the workgroups of all
// first stages come first in the grid, those of the second stages behind them.  A second-stage workgroup fetches its
// first sign words, then waits until its linear's h is complete (the hardware starts workgroups in the order of their
// ids, so every workgroup that is waited for is already running or done).
// Signalling, one slot of kFusedSlotWords words per launch, every counter and flag in a 128-byte line of its own:
// first-stage workgroups count their arrival per linear; the one that completes the count raises the linear's
// kFusedFlagLines ready flags, and a waiting workgroup polls one of them (1500 workgroups polling the arrival counter
// itself would queue every arrival behind their loads at one memory channel).  The last second-stage workgroup to
// finish puts the slot back to zero, so a slot serves launch after launch (and replay after replay of a captured
// launch) without being cleared from outside.
constexpr int kFusedMax = 8;
constexpr int kFusedFlagLines = 16;
constexpr int kFusedLineWords = 32;
constexpr int kFusedDoneLine = kFusedMax;                            // lines 0..7: arrivals per linear, 8: finished second stages
constexpr int kFusedFlagLine0 = 16;                                  // flag j of linear i: line 16 + i * kFusedFlagLines + j
constexpr int kFusedSlotLines = kFusedFlagLine0 + kFusedMax * kFusedFlagLines;
constexpr int kFusedSlotWords = kFusedSlotLines * kFusedLineWords;   // 18 KiB
struct FusedArgs {
    StageArgs a[kFusedMax];          // first stages
    StageArgs b[kFusedMax];          // second stages
    int first_a[kFusedMax + 1];      // first workgroup of every first stage; [kFusedMax] = their total
    int first_b[kFusedMax + 1];      // the same for the second stages, counted from the end of the first stages
    unsigned* slot;                  // kFusedSlotWords words, zero between launches
    unsigned* status;
    unsigned spin_limit;
};

template <int DT, int BATCH>
__global__ __launch_bounds__(256) void gemv_fused_kernel(FusedArgs f) {
    const int b = (int)blockIdx.x;
    const int n1 = f.first_a[kFusedMax];
    if (b < n1) {
        int i = 0;
#pragma unroll
        for (int k = 1; k < kFusedMax; ++k) i += b >= f.first_a[k] ? 1 : 0;
        stage_body<DT, true, BATCH, 1, true>(f.a[i], b - f.first_a[i], StageWait{});
        // every wavefront waits until its own stores of h have been acknowledged, the barrier collects all of them,
        // then the arrival is counted
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        if (threadIdx.x < kWave) {
            unsigned before = 0;
            if (threadIdx.x == 0)
                before = __hip_atomic_fetch_add(f.slot + i * kFusedLineWords, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            before = __builtin_amdgcn_readfirstlane(before);
            if (before + 1u == (unsigned)(f.first_a[i + 1] - f.first_a[i]) && threadIdx.x < kFusedFlagLines)
                __hip_atomic_store(f.slot + (kFusedFlagLine0 + i * kFusedFlagLines + (int)threadIdx.x) * kFusedLineWords, 1u,
                                   __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    } else {
        const int lb = b - n1;
        int i = 0;
#pragma unroll
        for (int k = 1; k < kFusedMax; ++k) i += lb >= f.first_b[k] ? 1 : 0;
        StageWait w;
        w.counter = f.slot + (kFusedFlagLine0 + i * kFusedFlagLines + (lb & (kFusedFlagLines - 1))) * kFusedLineWords;
        w.target = 1u;
        w.spin_limit = f.spin_limit;
        w.status = f.status;
        stage_body<DT, false, BATCH, 1, true>(f.b[i], lb - f.first_b[i], w);
        __syncthreads();
        if (threadIdx.x < kWave) {
            unsigned before = 0;
            if (threadIdx.x == 0)
                before = __hip_atomic_fetch_add(f.slot + kFusedDoneLine * kFusedLineWords, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            before = __builtin_amdgcn_readfirstlane(before);
            if (before + 1u == (unsigned)f.first_b[kFusedMax]) {     // everybody is past its wait: clear the slot for the next launch
                for (int k = (int)threadIdx.x; k < kFusedSlotLines; k += kWave)
                    __hip_atomic_store(f.slot + k * kFusedLineWords, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
        }
    }
}

// One stage of up to kFusedMax linears in one launch, no dependencies inside it: the grids of the linears one behind
// the other.  Two such launches (all first stages, all second stages) are what a group of independent linears costs.
struct GroupArgs {
    StageArgs s[kFusedMax];
    int first[kFusedMax + 1];        // first workgroup of every linear; [kFusedMax] = the grid
};

template <int DT, bool FIRST, int BATCH>
__global__ __launch_bounds__(256) void gemv_group_kernel(GroupArgs g) {
    const int b = (int)blockIdx.x;
    int i = 0;
#pragma unroll
    for (int k = 1; k < kFusedMax; ++k) i += b >= g.first[k] ? 1 : 0;
    stage_body<DT, FIRST, BATCH, 1, false>(g.s[i], b - g.first[i], StageWait{});
}

// ---- host side --------------------------------------------------------------------------------
static int pick_group_log2(int units, int rows, int batch, double grid_cap = 1536.0) {
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
            // more workgroups than stay resident run in rounds: beyond the cap a larger grid counts for less, not the same
            double grid = (double)rows / (4 * (kWave / G));
            if (grid > grid_cap) grid = grid_cap * (grid_cap / grid);
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

// Pieces of 8 and 16 batch rows go through the run-list kernel on this one stage (MFMA unit arithmetic: 1.5 and 2.5
// times faster there); smaller pieces are as fast or faster on the lane-group kernel below, whose launches carry less
// fixed cost.
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

// ---- fused launches ---------------------------------------------------------------------------
// The signalling slots live in a device array inside the library (zero when the module is loaded, put back to zero
// by every launch that used them): 256 slots of 18 KiB, dealt round robin to the calls.  Two calls collide on a slot
// only when they run at the same time on different streams AND are a multiple of 256 calls apart.
constexpr int kFusedSlots = 256;
static __device__ __align__(256) unsigned fused_counters[kFusedSlots * kFusedSlotWords];
static __device__ unsigned fused_status_word;
static std::atomic<unsigned> g_fused_ticket{0};
static unsigned* g_fused_counters_ptr[64];
static unsigned* g_fused_status_ptr[64];
static PerDeviceFlag g_fused_known;

static hipError_t fused_pointers(unsigned** counters, unsigned** status) {
    const int dev = current_device();
    if (dev < 0 || dev >= 64) return hipErrorInvalidDevice;
    if (!g_fused_known.test(dev)) {
        unsigned *c = nullptr, *st = nullptr;
        hipError_t e = hipGetSymbolAddress((void**)&c, HIP_SYMBOL(fused_counters));
        if (e != hipSuccess) return e;
        e = hipGetSymbolAddress((void**)&st, HIP_SYMBOL(fused_status_word));
        if (e != hipSuccess) return e;
        g_fused_counters_ptr[dev] = c;
        g_fused_status_ptr[dev] = st;
        g_fused_known.set(dev);
    }
    *counters = g_fused_counters_ptr[dev];
    *status = g_fused_status_ptr[dev];
    return hipSuccess;
}

int gemv_fused_max() { return kFusedMax; }

static std::atomic<unsigned> g_fused_spin_limit{0};
void gemv_fused_set_spin_limit(unsigned polls) { g_fused_spin_limit.store(polls); }

hipError_t gemv_fused_status(unsigned* out, hipStream_t stream) {
    unsigned *c = nullptr, *st = nullptr;
    hipError_t e = fused_pointers(&c, &st);
    if (e != hipSuccess) return e;
    e = hipMemcpyAsync(out, st, sizeof(unsigned), hipMemcpyDeviceToHost, stream);
    if (e != hipSuccess) return e;
    e = hipStreamSynchronize(stream);
    if (e == hipSuccess && *out != 0) {
        e = hipMemsetAsync(st, 0, sizeof(unsigned), stream);
        if (e == hipSuccess) e = hipStreamSynchronize(stream);
    }
    return e;
}

static void fill_stage(StageArgs& a, bool first, const uint32_t* bits, const void* in, const void* s_col, const void* s_row,
                       void* out, const void* bias, int batch, int rows, int words, int K, int in_stride, int out_stride,
                       double grid_cap) {
    a.bits = bits; a.in = in; a.out = out;
    a.bias = (const uint16_t*)bias; a.s_col = (const uint16_t*)s_col; a.s_row = (const uint16_t*)s_row;
    a.rows = rows; a.words = words; a.K = K; a.in_stride = in_stride; a.out_stride = out_stride;
    a.units = (words + 3) / 4;
    a.vec_bits = (words % 4 == 0) && aligned16(bits);
    const size_t in_elt = first ? 2 : 4;
    a.vec_in = aligned16(in) && ((size_t)in_stride * in_elt) % 16 == 0 && (!s_col || aligned16(s_col));
    a.addend = nullptr;
    a.out_f32 = first ? 1 : 0;
    int cap = (kLdsBudget - batch * kXsumBytesPerRow - batch * (int)sizeof(uint4)) / (batch * 16 * (int)sizeof(uint4));
    cap = (cap - 1) & ~1;
    if (cap > kXsumStride - 2) cap = kXsumStride - 2;
    a.chunk_units = a.units < cap ? a.units : cap;
    a.group_log2 = pick_group_log2(a.chunk_units, rows, batch, grid_cap);
}

// Workgroups that the lane-group choice of a group launch aims at, shared out by packed words (a single linear aims at
// 1536): fewer, larger workgroups stage the input vectors less often (Llama-2-7B layer at batch 1 as {q,k,v} {o}
// {gate,up} {down}: 53 us per layer at 1536, 48.5 at 512 .. 768, 50.7 at 384).
constexpr double kGroupGridCap = 768.0;

// y_i = s_out_i * (U_i (s_mid_i * (Vt_i (s_in_i * x_i)))) for `count` independent linears (<= gemv_fused_max());
// batch 1, 2 or 4 rows; h_i: fp32 [batch, r_i] scratch of the caller.  Two launches (all first stages, then all second
// stages), or with `one_launch` a single one whose second-stage workgroups wait inside the kernel.
hipError_t gemv_fused(int dtype, int count, int batch, const void* const* x, const void* const* s_in,
                      const uint32_t* const* vt_bits, const void* const* s_mid, const uint32_t* const* u_bits,
                      const void* const* s_out, const void* const* bias, float* const* h, void* const* y,
                      const int* n, const int* r, const int* m, bool one_launch, hipStream_t stream) {
    if (count < 1 || count > kFusedMax || (batch != 1 && batch != 2 && batch != 4)) return hipErrorInvalidValue;
    FusedArgs f;
    size_t lds_a = 0, lds_b = 0;
    int na = 0, nb = 0;
    // every linear gets the share of the resident workgroups that its packed words have in the stage
    double words_a = 0.0, words_b = 0.0;
    for (int i = 0; i < count; ++i) {
        words_a += (double)r[i] * ((n[i] + 31) / 32);
        words_b += (double)m[i] * ((r[i] + 31) / 32);
    }
    for (int i = 0; i < kFusedMax; ++i) {
        const int q = i < count ? i : count - 1;
        const double cap_a = kGroupGridCap * ((double)r[q] * ((n[q] + 31) / 32)) / (words_a > 0 ? words_a : 1.0);
        const double cap_b = kGroupGridCap * ((double)m[q] * ((r[q] + 31) / 32)) / (words_b > 0 ? words_b : 1.0);
        fill_stage(f.a[i], true, vt_bits[q], x[q], s_in[q], s_mid[q], h[q], nullptr, batch, r[q], (n[q] + 31) / 32, n[q], n[q], r[q],
                   cap_a < 64.0 ? 64.0 : cap_a);
        fill_stage(f.b[i], false, u_bits[q], h[q], nullptr, s_out[q], y[q], bias ? bias[q] : nullptr, batch, m[q], (r[q] + 31) / 32,
                   r[q], r[q], m[q], cap_b < 64.0 ? 64.0 : cap_b);
        f.first_a[i] = na;
        f.first_b[i] = nb;
        if (i < count) {
            for (const StageArgs* st : {&f.a[i], &f.b[i]}) {
                const int rows_per_block = 4 * (kWave >> st->group_log2);
                const int blocks = (st->rows + rows_per_block - 1) / rows_per_block;
                const size_t need = (size_t)batch * kXsumBytesPerRow + (size_t)xs_chunks(batch, st->chunk_units | 1) * sizeof(uint4);
                if (st == &f.a[i]) { na += blocks; if (need > lds_a) lds_a = need; }
                else { nb += blocks; if (need > lds_b) lds_b = need; }
            }
        }
    }
    f.first_a[kFusedMax] = na;
    f.first_b[kFusedMax] = nb;
    if (na == 0 || nb == 0) return hipSuccess;
    const int dev = current_device();
    const int bi = batch == 1 ? 0 : batch == 2 ? 1 : 2;
    auto raise_lds = [&](auto kern, size_t lds_bytes, PerDeviceFlag& attr_done) -> hipError_t {
        if (lds_bytes > 64 * 1024 && !attr_done.test(dev)) {
            hipError_t err = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, kLdsBudget);
            if (err != hipSuccess) return err;
            attr_done.set(dev);
        }
        return hipSuccess;
    };
    if (!one_launch) {
        GroupArgs ga, gb;
        for (int i = 0; i < kFusedMax; ++i) { ga.s[i] = f.a[i]; gb.s[i] = f.b[i]; }
        for (int i = 0; i <= kFusedMax; ++i) { ga.first[i] = f.first_a[i]; gb.first[i] = f.first_b[i]; }
        auto launch = [&](auto kern, const GroupArgs& g, int grid, size_t lds_bytes, PerDeviceFlag& attr_done) -> hipError_t {
            hipError_t err = raise_lds(kern, lds_bytes, attr_done);
            if (err != hipSuccess) return err;
            hipLaunchKernelGGL(kern, dim3(grid), dim3(256), lds_bytes, stream, g);
            return hipGetLastError();
        };
        static PerDeviceFlag done[2][2][3];
        hipError_t e;
#define NQ_GROUP_LAUNCH(DT, B)                                                                     \
        e = launch(gemv_group_kernel<DT, true, B>, ga, na, lds_a, done[DT][0][bi]);                \
        if (e == hipSuccess) e = launch(gemv_group_kernel<DT, false, B>, gb, nb, lds_b, done[DT][1][bi]);
        if (dtype == 0) {
            if (batch == 1) { NQ_GROUP_LAUNCH(0, 1) } else if (batch == 2) { NQ_GROUP_LAUNCH(0, 2) } else { NQ_GROUP_LAUNCH(0, 4) }
        } else {
            if (batch == 1) { NQ_GROUP_LAUNCH(1, 1) } else if (batch == 2) { NQ_GROUP_LAUNCH(1, 2) } else { NQ_GROUP_LAUNCH(1, 4) }
        }
#undef NQ_GROUP_LAUNCH
        return e;
    }
    unsigned *counters = nullptr, *status = nullptr;
    hipError_t e = fused_pointers(&counters, &status);
    if (e != hipSuccess) return e;
    f.slot = counters + (size_t)(g_fused_ticket.fetch_add(1u) % kFusedSlots) * kFusedSlotWords;
    f.status = status;
    const unsigned spin = g_fused_spin_limit.load();
    f.spin_limit = spin ? spin : (1u << 20);
    const size_t lds_bytes = lds_a > lds_b ? lds_a : lds_b;
    auto launch = [&](auto kern, PerDeviceFlag& attr_done) -> hipError_t {
        hipError_t err = raise_lds(kern, lds_bytes, attr_done);
        if (err != hipSuccess) return err;
        hipLaunchKernelGGL(kern, dim3(na + nb), dim3(256), lds_bytes, stream, f);
        return hipGetLastError();
    };
    static PerDeviceFlag done[2][3];
    if (dtype == 0) {
        if (batch == 1) return launch(gemv_fused_kernel<0, 1>, done[0][bi]);
        if (batch == 2) return launch(gemv_fused_kernel<0, 2>, done[0][bi]);
        return launch(gemv_fused_kernel<0, 4>, done[0][bi]);
    }
    if (batch == 1) return launch(gemv_fused_kernel<1, 1>, done[1][bi]);
    if (batch == 2) return launch(gemv_fused_kernel<1, 2>, done[1][bi]);
    return launch(gemv_fused_kernel<1, 4>, done[1][bi]);
}

}  // namespace nq
