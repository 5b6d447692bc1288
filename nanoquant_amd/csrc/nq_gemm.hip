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
// integer logic only.  With an input scale the operand is +-s_in[k] instead of +-1 (the scale pair
// XOR the sign bits), so x * s_in is formed exactly inside the MFMA and staging stays a plain copy.
// Activations are the A operand and come from an LDS slab shared by the four wavefronts of a
// workgroup; accumulation is fp32 in the MFMA accumulators.  With A = activations the result registers of a lane run along the output row index,
// which makes the epilogue stores contiguous.
//
// Work split: grid.x = 128-row blocks (4 wavefronts x 32 rows), grid.y = token blocks of 32*TT,
// grid.z = k-splits.  With one k-split the epilogue scales and stores directly; otherwise partial
// sums are added into an fp32 scratch with hardware float atomics and a small second kernel scales
// and converts (and re-zeroes the scratch, which must be zero on entry).
#include "nq_common.h"
#include "nq_kernels.h"
#include "nq_mfma.h"

namespace nq {

struct GemmArgs {
    const void* x;          // [T, K] 16-bit
    const uint4* tiles;     // [R/32][K/256][64 lanes] 16 bytes each
    const uint16_t* s_in;   // [K] or null
    const uint16_t* s_out;  // [R] or null
    const uint16_t* bias;   // [R] added after the output scale, or null
    void* y;                // [T, R] 16-bit
    float* acc;             // [T, R] fp32 partial sums (k-split only)
    int T, K, R;
    int ktiles;             // K / 256
    int ktiles_per_split;
    int xcd_gx;             // > 0: flat grid, token blocks dealt to the 8 XCDs; value = row blocks
};

// Issues the global loads of one activation slab [32*TT tokens][KS k] starting at k0 (and its KS input
// scales) into registers; nothing waits on them here.
template <int TT, int KS, bool SCALED>
__device__ __forceinline__ void fetch_slab(const GemmArgs& a, int tok0, int k0, u32x4_t (&xr)[TT * KS / 64], uint32_t& sr) {
    constexpr int kChunks = KS / 8;   // 16-byte chunks per token row
#pragma unroll
    for (int pass = 0; pass < TT * KS / 64; ++pass) {
        const int q = pass * 256 + threadIdx.x;
        // rows beyond T repeat the last token; their results are never stored
        const int tok = min(tok0 + q / kChunks, a.T - 1), c8 = (q % kChunks) * 8;
        xr[pass] = *(const u32x4_t*)((const uint16_t*)a.x + (size_t)tok * a.K + k0 + c8);
    }
    if constexpr (SCALED) {
        if (threadIdx.x < KS / 2) sr = *(const uint32_t*)(a.s_in + k0 + 2 * threadIdx.x);
    }
}

// TT: 32-token tiles per wavefront, RT: 32-row tiles per wavefront, KS: k-values per LDS slab (128 or
// 256).  A workgroup of 4 wavefronts covers 32*TT tokens x 128*RT rows.
template <int DT, int TT, int RT, int KS, bool SPLIT, bool SCALED>
__device__ __forceinline__ void block_tile(const GemmArgs& a, int bx, int by, int bz) {
    using E = Elem<DT>;
    constexpr int kPitch = slab_pitch<KS>();
    constexpr int kSubs = kTileK / KS;       // slabs per weight tile
    constexpr int kPasses = TT * KS / 64;    // 16-byte chunks each thread stages per slab
    extern __shared__ uint16_t slab[];       // [32*TT][kPitch], then the KS input scales of the slab
    uint16_t* scale_lds = slab + 32 * TT * kPitch;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int rt = (bx * 4 + wave) * RT;           // first of the RT 32-row tiles of this wavefront
    const bool have_rows = rt * 32 < a.R;
    const int ntiles = min(RT, a.R / 32 - rt);     // R % 32 == 0
    const int tok0 = by * (32 * TT);
    const int kt_begin = bz * a.ktiles_per_split;
    const int kt_end = min(kt_begin + a.ktiles_per_split, a.ktiles);

    float16_t acc[RT][TT];
#pragma unroll
    for (int r = 0; r < RT; ++r)
#pragma unroll
        for (int tt = 0; tt < TT; ++tt)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[r][tt][v] = 0.f;

    const uint4* tile_ptr = a.tiles + ((size_t)rt * a.ktiles + kt_begin) * 64 + lane;
    const size_t tile_pitch = (size_t)a.ktiles * 64;   // uint4 elements between consecutive row tiles
    uint4 wnext[RT];
#pragma unroll
    for (int r = 0; r < RT; ++r) {
        wnext[r] = make_uint4(0, 0, 0, 0);
        if (r < ntiles && kt_begin < kt_end) wnext[r] = tile_ptr[r * tile_pitch];
    }

    // The next slab travels global -> registers while the MFMAs of the current one run, and registers
    // -> LDS between the two barriers at the top of the next step.
    u32x4_t xr[kPasses];
    uint32_t sr = 0;
    if (kt_begin < kt_end) fetch_slab<TT, KS, SCALED>(a, tok0, kt_begin * kTileK, xr, sr);

#pragma unroll 1
    for (int kt = kt_begin; kt < kt_end; ++kt) {
        uint4 w[RT];
#pragma unroll
        for (int r = 0; r < RT; ++r) {
            w[r] = wnext[r];
            if (r < ntiles && kt + 1 < kt_end) wnext[r] = tile_ptr[r * tile_pitch + (size_t)(kt + 1 - kt_begin) * 64];
        }
#pragma unroll
        for (int sub = 0; sub < kSubs; ++sub) {
            if (sub != 0 || kt != kt_begin) __syncthreads();
#pragma unroll
            for (int pass = 0; pass < kPasses; ++pass) {
                const int q = pass * 256 + threadIdx.x;
                *(u32x4_t*)(slab + (q / (KS / 8)) * kPitch + (q % (KS / 8)) * 8) = xr[pass];
            }
            if constexpr (SCALED) {
                if (threadIdx.x < KS / 2) *(uint32_t*)(scale_lds + 2 * threadIdx.x) = sr;
            }
            __syncthreads();
            if (sub + 1 < kSubs) fetch_slab<TT, KS, SCALED>(a, tok0, kt * kTileK + (sub + 1) * KS, xr, sr);
            else if (kt + 1 < kt_end) fetch_slab<TT, KS, SCALED>(a, tok0, (kt + 1) * kTileK, xr, sr);

            // wavefronts beyond the last row tile run on zero words; nothing of theirs is stored
#pragma unroll
            for (int t = 0; t < KS / 16; ++t) {
                const int tg = sub * (KS / 16) + t;   // 16-k step within the weight tile
                const int s = 4 * (tg & 3);
                uint4 sp;
                if constexpr (SCALED) sp = *(const uint4*)(scale_lds + 16 * t + 8 * (lane >> 5));   // broadcast read
                uint4 bfrag[RT];
#pragma unroll
                for (int r = 0; r < RT; ++r) {
                    const uint32_t word = comp4(w[r], tg >> 2);
                    if constexpr (SCALED) {
                        // +-s_in[k]: the scale pair with its sign bits flipped by the packed bits, so that
                        // x * s_in is formed exactly inside the MFMA (the reference folds s_in into its
                        // dequantised fragment the same way, gemm_kernel.cu:231-237)
                        bfrag[r].x = sp.x ^ ((word << (s + 0)) & kSignPair);
                        bfrag[r].y = sp.y ^ ((word << (s + 1)) & kSignPair);
                        bfrag[r].z = sp.z ^ ((word << (s + 2)) & kSignPair);
                        bfrag[r].w = sp.w ^ ((word << (s + 3)) & kSignPair);
                    } else {
                        bfrag[r].x = ((word << (s + 0)) & kSignPair) | E::kOnePair;
                        bfrag[r].y = ((word << (s + 1)) & kSignPair) | E::kOnePair;
                        bfrag[r].z = ((word << (s + 2)) & kSignPair) | E::kOnePair;
                        bfrag[r].w = ((word << (s + 3)) & kSignPair) | E::kOnePair;
                    }
                }
#pragma unroll
                for (int tt = 0; tt < TT; ++tt) {
                    const uint4 afrag = *(const uint4*)(slab + (tt * 32 + (lane & 31)) * kPitch + 16 * t + 8 * (lane >> 5));
#pragma unroll
                    for (int r = 0; r < RT; ++r) acc[r][tt] = Mfma<DT>::run(afrag, bfrag[r], acc[r][tt]);
                }
            }
        }
    }

    if (!have_rows) return;
#pragma unroll
    for (int r = 0; r < RT; ++r) {
        if (r >= ntiles) break;
        const int row = (rt + r) * 32 + (lane & 31);
        float sc = 1.f, bs = 0.f;
        if (!SPLIT && a.s_out) sc = E::to_float(a.s_out[row]);
        if (!SPLIT && a.bias) bs = E::to_float(a.bias[row]);
#pragma unroll
        for (int tt = 0; tt < TT; ++tt) {
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int tok = tok0 + tt * 32 + 8 * (v >> 2) + 4 * (lane >> 5) + (v & 3);
                if (tok < a.T) {
                    const size_t o = (size_t)tok * a.R + row;
                    if (SPLIT) atomicAdd(a.acc + o, acc[r][tt][v]);
                    else ((uint16_t*)a.y)[o] = E::from_float_sat(acc[r][tt][v] * sc + bs);
                }
            }
        }
    }
}

template <int DT, int TT, int RT, int KS, bool SPLIT, bool SCALED>
__global__ __launch_bounds__(256) void gemm_onebit_kernel(GemmArgs a) {
    // Workgroups go to the 8 XCDs round-robin by linear id.  With the flat grid every XCD owns the token
    // blocks y = xcd (mod 8), so the workgroups that share an activation slab also share an L2.
    int bx = blockIdx.x, by = blockIdx.y;
    if (a.xcd_gx > 0) {
        const int slot = blockIdx.x >> 3;
        by = (slot / a.xcd_gx) * 8 + (blockIdx.x & 7);
        bx = slot % a.xcd_gx;
        if (by * (32 * TT) >= a.T) return;
    }
    block_tile<DT, TT, RT, KS, SPLIT, SCALED>(a, bx, by, blockIdx.z);
}

// Few tokens: one 32-row x 32-token output tile per workgroup, the four wavefronts split k among them
// (wavefront w takes the weight tiles w, w+4, ...) and add their accumulators through LDS at the end.
// No global atomics, no scratch, no second launch; R/32 x T/32 workgroups, and the wavefronts of a workgroup
// never wait for each other inside the k loop (each stages its own activation slab).
template <int DT, bool SCALED, int RT>
__device__ __forceinline__ void kwave_tile(const GemmArgs& a, int row_block, int token_block) {
    using E = Elem<DT>;
    constexpr int kPitch = slab_pitch<kTileK>();
    constexpr int kSlabHalves = 32 * kPitch + kTileK;            // slab + its 256 input scales
    extern __shared__ uint16_t slabs[];                          // [4 wavefronts][kSlabHalves]
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    uint16_t* slab = slabs + wave * kSlabHalves;
    uint16_t* scale_lds = slab + 32 * kPitch;
    const int rt = row_block * RT;                               // first of the RT 32-row tiles of this workgroup
    const int ntiles = min(RT, a.R / 32 - rt);
    const int tok0 = token_block * 32;

    float16_t acc[RT];
#pragma unroll
    for (int r = 0; r < RT; ++r)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[r][v] = 0.f;

    // the wavefront's slab: 32 tokens x 256 k = 1024 16-byte chunks, 16 per lane
    u32x4_t xr[16];
    u32x4_t sr;                                                  // 8 of the 256 scales per lane (lanes 0..31)
    auto fetch = [&](int kt) {
        const int k0 = kt * kTileK;
#pragma unroll
        for (int pass = 0; pass < 16; ++pass) {
            const int q = pass * 64 + lane;
            const int tok = min(tok0 + (q >> 5), a.T - 1), c8 = (q & 31) * 8;   // rows beyond T repeat the last token
            xr[pass] = *(const u32x4_t*)((const uint16_t*)a.x + (size_t)tok * a.K + k0 + c8);
        }
        if constexpr (SCALED) sr = *(const u32x4_t*)(a.s_in + k0 + 8 * (lane & 31));
    };

    const uint4* tile_ptr = a.tiles + (size_t)rt * a.ktiles * 64 + lane;
    const size_t tile_pitch = (size_t)a.ktiles * 64;             // uint4 elements between consecutive row tiles
    uint4 wnext[RT];
#pragma unroll
    for (int r = 0; r < RT; ++r) wnext[r] = make_uint4(0, 0, 0, 0);
    if (wave < a.ktiles) {
#pragma unroll
        for (int r = 0; r < RT; ++r)
            if (r < ntiles) wnext[r] = tile_ptr[r * tile_pitch + (size_t)wave * 64];
        fetch(wave);
    }
#pragma unroll 1
    for (int kt = wave; kt < a.ktiles; kt += 4) {
        // registers -> own slab; LDS operations of one wavefront complete in order, no barrier needed
#pragma unroll
        for (int pass = 0; pass < 16; ++pass) {
            const int q = pass * 64 + lane;
            *(u32x4_t*)(slab + (q >> 5) * kPitch + (q & 31) * 8) = xr[pass];
        }
        if constexpr (SCALED) {
            if (lane < 32) *(u32x4_t*)(scale_lds + 8 * lane) = sr;
        }
        uint4 w[RT];
#pragma unroll
        for (int r = 0; r < RT; ++r) w[r] = wnext[r];
        if (kt + 4 < a.ktiles) {
#pragma unroll
            for (int r = 0; r < RT; ++r)
                if (r < ntiles) wnext[r] = tile_ptr[r * tile_pitch + (size_t)(kt + 4) * 64];
            fetch(kt + 4);
        }
#pragma unroll
        for (int t = 0; t < 16; ++t) {
            const int s = 4 * (t & 3);
            uint4 sp;
            if constexpr (SCALED) sp = *(const uint4*)(scale_lds + 16 * t + 8 * (lane >> 5));
            const uint4 afrag = *(const uint4*)(slab + (lane & 31) * kPitch + 16 * t + 8 * (lane >> 5));
#pragma unroll
            for (int r = 0; r < RT; ++r) {
                const uint32_t word = comp4(w[r], t >> 2);
                uint4 bfrag;
                if constexpr (SCALED) {
                    bfrag.x = sp.x ^ ((word << (s + 0)) & kSignPair);
                    bfrag.y = sp.y ^ ((word << (s + 1)) & kSignPair);
                    bfrag.z = sp.z ^ ((word << (s + 2)) & kSignPair);
                    bfrag.w = sp.w ^ ((word << (s + 3)) & kSignPair);
                } else {
                    bfrag.x = ((word << (s + 0)) & kSignPair) | E::kOnePair;
                    bfrag.y = ((word << (s + 1)) & kSignPair) | E::kOnePair;
                    bfrag.z = ((word << (s + 2)) & kSignPair) | E::kOnePair;
                    bfrag.w = ((word << (s + 3)) & kSignPair) | E::kOnePair;
                }
                acc[r] = Mfma<DT>::run(afrag, bfrag, acc[r]);
            }
        }
    }

    // ---- add the four partial tiles through LDS (the slabs are free now) ----
    __syncthreads();
    // [RT][4][16] rows of kPartPitch floats; lane l of a row sits at (l & 31) + 33 * (l >> 5).  Pitch 66 and the
    // odd offset of the upper half make both the stores here and the gathering loads below free of bank conflicts
    // (the plain [..][64] layout put the 64 gathering lanes on 4 banks: 3600 conflict cycles per workgroup).
    constexpr int kPartPitch = 66;
    static_assert(RT * 4 * 16 * kPartPitch * sizeof(float) <= 4 * kSlabHalves * sizeof(uint16_t), "partial tiles must fit the slabs");
    float* part = (float*)slabs;                                 // RT x 16.25 KiB <= the slabs' 68 KiB
#pragma unroll
    for (int r = 0; r < RT; ++r)
#pragma unroll
        for (int v = 0; v < 16; ++v) part[((r * 4 + wave) * 16 + v) * kPartPitch + (lane & 31) + 33 * (lane >> 5)] = acc[r][v];
    __syncthreads();
    // Thread (token t, row octet o) of each half of the workgroup sums the four partial values of 8 consecutive
    // rows and stores them as one 16-byte chunk; the two halves take the row tiles in turn (one half idles when
    // there is only one).  Accumulator element v of lane l is token 8*(v>>2) + 4*(l>>5) + (v&3), row l&31.
    {
        const int th = threadIdx.x & 127, first_r = threadIdx.x >> 7;
        const int t = th >> 2, o = th & 3;
        const int v = 4 * (t >> 3) + (t & 3), l0 = 33 * ((t >> 2) & 1) + 8 * o;   // lanes 32 h + 8 o + j of the tile row
        const int tok = tok0 + t;
#pragma unroll
        for (int r = first_r; r < RT; r += 2) {
            if (r >= ntiles) break;
            const int row0 = (rt + r) * 32 + 8 * o;
            const float* pr = part + (size_t)r * 4 * 16 * kPartPitch;
            float sums[8];
#pragma unroll
            for (int j = 0; j < 8; ++j)
                sums[j] = (pr[(0 * 16 + v) * kPartPitch + l0 + j] + pr[(1 * 16 + v) * kPartPitch + l0 + j]) +
                          (pr[(2 * 16 + v) * kPartPitch + l0 + j] + pr[(3 * 16 + v) * kPartPitch + l0 + j]);
            u32x4_t sc = {E::kOnePair, E::kOnePair, E::kOnePair, E::kOnePair};
            u32x4_t bs = {0u, 0u, 0u, 0u};
            if (a.s_out) sc = *(const u32x4_t*)(a.s_out + row0);
            if (a.bias) bs = *(const u32x4_t*)(a.bias + row0);
            u32x4_t outv;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const uint32_t sw = sc[j], bw = bs[j];
                const uint16_t lo = E::from_float_sat(sums[2 * j] * E::to_float((uint16_t)(sw & 0xFFFFu)) + E::to_float((uint16_t)(bw & 0xFFFFu)));
                const uint16_t hi = E::from_float_sat(sums[2 * j + 1] * E::to_float((uint16_t)(sw >> 16)) + E::to_float((uint16_t)(bw >> 16)));
                outv[j] = (uint32_t)lo | ((uint32_t)hi << 16);
            }
            if (tok < a.T) *(u32x4_t*)((uint16_t*)a.y + (size_t)tok * a.R + row0) = outv;
        }
    }
}

template <int DT, bool SCALED, int RT>
__global__ __launch_bounds__(256) void gemm_kwave_kernel(GemmArgs a) {
    kwave_tile<DT, SCALED, RT>(a, blockIdx.x, blockIdx.y);
}

// Several GEMMs of the few-token kind in one launch (the projections that share a layer's tokens): workgroup b
// belongs to the problem p with first[p] <= b < first[p + 1]; inside a problem the row blocks run fastest, so
// neighbours share an activation slab.  All problems have the same token count.
constexpr int kGroupMax = 16;   // 16 problems of 80 bytes: well inside the 4 KB of kernel arguments
struct GemmGroup {
    GemmArgs a[kGroupMax];
    int first[kGroupMax + 1];
    int count;
};

template <int DT, bool SCALED, int RT>
__global__ __launch_bounds__(256) void gemm_kwave_group_kernel(GemmGroup g) {
    const int b = blockIdx.x;
    // first[i] of the unused entries is the grid size, so no count is needed; all of first[] comes with one load
    int p = 0;
#pragma unroll
    for (int i = 1; i < kGroupMax; ++i) p += b >= g.first[i] ? 1 : 0;
    const GemmArgs a = g.a[p];
    const int local = b - g.first[p];
    const int gx = (a.R / 32 + RT - 1) / RT;
    kwave_tile<DT, SCALED, RT>(a, local % gx, local / gx);
}

// The same for more tokens (above kKwaveGroupMaxTokens): block tiles of 64 tokens x 128*RT rows, every workgroup walks the whole k of
// its problem (no k-split, no scratch).  Workgroups go to the 8 XCDs round-robin by id and first[p] is a multiple
// of 8, so (id - first[p]) mod 8 is the XCD; the mapping keeps the workgroups that share an activation slab on one
// XCD (one L2) where the number of token blocks gy allows it: gy a multiple of 8 (or large): XCD = token block
// mod 8; gy = 1, 2, 4: XCD x owns token block x mod gy and every (8/gy)-th row block; otherwise row blocks run
// fastest.  a.xcd_gx holds the number of row blocks; group_blocks() is the host's count for the same mapping.
__host__ __device__ inline int group_mode(int gy) { return (gy % 8 == 0 || gy >= 32) ? 0 : (8 % gy == 0) ? 1 : 2; }
static int group_blocks(int gx, int gy) {
    const int mode = group_mode(gy);
    if (mode == 0) return gx * ((gy + 7) / 8 * 8);
    if (mode == 1) { const int sub = 8 / gy; return (gx + sub - 1) / sub * 8; }
    return (gx * gy + 7) / 8 * 8;
}
template <int DT, int RT, bool SCALED>
__global__ __launch_bounds__(256) void gemm_block_group_kernel(GemmGroup g) {
    const int b = blockIdx.x;
    int p = 0;
    while (p + 1 < g.count && b >= g.first[p + 1]) ++p;
    const GemmArgs a = g.a[p];
    const int local = b - g.first[p];
    const int gx = a.xcd_gx, gy = (a.T + 63) >> 6;
    const int mode = group_mode(gy);
    int bx, by;
    if (mode == 0) {
        const int slot = local >> 3;
        by = (slot / gx) * 8 + (local & 7);
        bx = slot % gx;
    } else if (mode == 1) {
        const int sub = 8 / gy, xcd = local & 7;
        by = xcd % gy;
        bx = (local >> 3) * sub + xcd / gy;
    } else {
        bx = local % gx;
        by = local / gx;
    }
    if (bx >= gx || by >= gy) return;
    block_tile<DT, 2, RT, kTileK, false, SCALED>(a, bx, by, 0);
}

// Scales, converts and stores the accumulated sums, and puts the accumulator back to zero: the scratch
// is zero on entry of every GEMM call and zero again when the call has finished.
template <int DT>
__global__ __launch_bounds__(256) void gemm_finish_kernel(float4* acc, const uint16_t* s_out, const uint16_t* bias, uint16_t* y, int R,
                                                          size_t n4) {
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
        float b0 = 0.f, b1 = 0.f, b2 = 0.f, b3 = 0.f;
        if (bias) {
            b0 = E::to_float(bias[row]); b1 = E::to_float(bias[row + 1]);
            b2 = E::to_float(bias[row + 2]); b3 = E::to_float(bias[row + 3]);
        }
        uint2 o;
        o.x = (uint32_t)E::from_float_sat(v.x * s0 + b0) | ((uint32_t)E::from_float_sat(v.y * s1 + b1) << 16);
        o.y = (uint32_t)E::from_float_sat(v.z * s2 + b2) | ((uint32_t)E::from_float_sat(v.w * s3 + b3) << 16);
        ((uint2*)y)[i] = o;
    }
}

// ---- host side --------------------------------------------------------------------------------
struct GemmPlan {
    int tt;       // 32-token tiles per wavefront
    int rt;       // 32-row tiles per wavefront
    int gx, gy, ksplit, ktiles_per_split;
    bool xcd;     // flat, XCD-aware grid
    bool kwave;   // few tokens: gemm_kwave_kernel (32x32 output tiles, wavefronts split k)
};

constexpr int kKwaveMaxTokens = 256;
// In a group the few-token tiles stay ahead a little longer (Llama-2-7B layer, share of the fp16 peak, few-token vs
// block tiles: 144 tokens 22.5 vs 19.6 %, 160 tokens 27.1 vs 22.3 %, 192 tokens 25.8 vs 26.1 %, 256 tokens 28.1 vs 30.8 %).
constexpr int kKwaveGroupMaxTokens = 160;

static GemmPlan plan_gemm(int T, int K, int R) {
    GemmPlan p;
    p.kwave = false;
    // A long k (more than 16 tiles) needs a k-split with atomics and a finish launch on block tiles, while the
    // wavefronts of a few-token tile split k for free: those GEMMs stay on few-token tiles up to 1024 tokens
    // (the two kernels cross at 2048 tokens for k 11008 -> 3072 rows).
    if (T <= kKwaveMaxTokens || (K / kTileK > 16 && T <= 1024)) {
        // 32x32 output tiles, wavefronts split k: no k-split scratch, one launch.  For the linears of a Llama-2-7B
        // layer one after the other these tiles are ahead of the block tiles up to 256 tokens, behind from 288 on.
        p.kwave = true;
        p.tt = 1; p.gy = (T + 31) / 32;
        // Every 32-row tile re-reads the 32-token activation slab, so wider workgroups save L2 traffic: with a
        // long k the widest that still leaves workgroups for three quarters of the CUs.  With a short k a workgroup
        // is gone before its neighbours have started, and more of them do better: two per CU there.
        const int min_workgroups = K / kTileK >= 16 ? 192 : 512;
        p.rt = 1;
        for (int rt = 2; rt <= 4; rt *= 2)
            if ((long)((R / 32 + rt - 1) / rt) * p.gy >= min_workgroups) p.rt = rt;
        p.gx = (R / 32 + p.rt - 1) / p.rt;
        p.ktiles_per_split = K / kTileK; p.ksplit = 1; p.xcd = false;
        return p;
    }
    // 64-token blocks measured faster than 128-token blocks at every token count tried (128 .. 4096):
    // more workgroups, fewer registers, three wavefronts per SIMD.  Two row tiles per wavefront halve the
    // LDS reads per MFMA and win once that still leaves two workgroups for every CU.
    p.tt = 2;
    {
        // Few tokens: 32-token blocks give twice the workgroups, which can spare the k-split and with it
        // the atomics and the finish launch (4096x4096 at 256 tokens: 44 -> 27 us per linear).  Only when
        // k is short enough for one workgroup to walk it (<= 16 tiles).
        const int gx1 = (R + 127) / 128, gy1 = (T + 31) / 32;
        if (gx1 * ((T + 63) / 64) < 512 && gx1 * gy1 >= 128 && K / kTileK <= 16) {
            p.tt = 1; p.rt = 1; p.gx = gx1; p.gy = gy1;
            p.ktiles_per_split = K / kTileK; p.ksplit = 1; p.xcd = false;
            return p;
        }
    }
    p.gy = (T + 32 * p.tt - 1) / (32 * p.tt);
    p.rt = ((R + 255) / 256) * p.gy >= 512 ? 2 : 1;
    p.gx = (R + 128 * p.rt - 1) / (128 * p.rt);
    const int ktiles = K / kTileK;
    int want = 512 / (p.gx * p.gy);          // k-splits needed to put two workgroups on every CU
    if (want < 1) want = 1;
    int max_split = ktiles / 2;              // keep at least 512 k per split
    if (max_split < 1) max_split = 1;
    int ks = want < max_split ? want : max_split;
    p.ktiles_per_split = (ktiles + ks - 1) / ks;
    p.ksplit = (ktiles + p.ktiles_per_split - 1) / p.ktiles_per_split;
    // the XCD-aware flat grid needs token blocks in multiples of 8 (or many of them) to stay balanced
    p.xcd = p.ksplit == 1 && (p.gy % 8 == 0 || p.gy >= 32);
    return p;
}

size_t gemm_scratch_bytes(int T, int K, int R) {
    if (T <= 0 || K <= 0 || R <= 0 || K % kTileK != 0) return 0;
    const GemmPlan p = plan_gemm(T, K, R);
    return p.ksplit > 1 ? (size_t)T * R * sizeof(float) : 0;
}

template <int DT, int TT, int RT, int KS, bool SPLIT, bool SCALED>
static hipError_t launch_variant(const GemmArgs& a, dim3 grid, size_t lds, hipStream_t stream) {
    auto kern = gemm_onebit_kernel<DT, TT, RT, KS, SPLIT, SCALED>;
    static PerDeviceFlag attr_done;              // per template instance and device
    const int dev = current_device();
    if (lds > 64 * 1024 && !attr_done.test(dev)) {
        hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return e;
        attr_done.set(dev);
    }
    hipLaunchKernelGGL(kern, grid, dim3(256), lds, stream, a);
    return hipSuccess;
}

template <int DT, int TT, int RT, int KS>
static hipError_t launch_gemm(const GemmArgs& a, const GemmPlan& p, hipStream_t stream) {
    const size_t lds = ((size_t)32 * TT * slab_pitch<KS>() + KS) * sizeof(uint16_t);
    dim3 grid(p.gx, p.gy, p.ksplit);
    if (p.xcd) grid = dim3(p.gx * ((p.gy + 7) / 8 * 8), 1, 1);
    const bool scaled = a.s_in != nullptr;
    hipError_t e;
    if (p.ksplit > 1) {
        e = scaled ? launch_variant<DT, TT, RT, KS, true, true>(a, grid, lds, stream)
                   : launch_variant<DT, TT, RT, KS, true, false>(a, grid, lds, stream);
        if (e != hipSuccess) return e;
        const size_t n4 = (size_t)a.T * a.R / 4;
        size_t zb = (n4 + 255) / 256;
        if (zb > 2048) zb = 2048;
        hipLaunchKernelGGL(gemm_finish_kernel<DT>, dim3((unsigned)zb), dim3(256), 0, stream, (float4*)a.acc, a.s_out,
                           a.bias, (uint16_t*)a.y, a.R, n4);
    } else {
        e = scaled ? launch_variant<DT, TT, RT, KS, false, true>(a, grid, lds, stream)
                   : launch_variant<DT, TT, RT, KS, false, false>(a, grid, lds, stream);
        if (e != hipSuccess) return e;
    }
    return hipGetLastError();
}

// Shapes must satisfy K % 256 == 0 and R % 32 == 0 (checked by the caller).  `scratch` (when
// gemm_scratch_bytes > 0) must be zero on entry and is zero again when the enqueued work has finished.
hipError_t gemm_onebit(int dtype, const void* x, const uint32_t* tiles, const void* s_in, const void* s_out,
                       void* y, float* scratch, int T, int K, int R, hipStream_t stream, const void* bias) {
    GemmArgs a;
    a.x = x; a.tiles = (const uint4*)tiles;
    a.s_in = (const uint16_t*)s_in; a.s_out = (const uint16_t*)s_out; a.bias = (const uint16_t*)bias;
    a.y = y; a.acc = scratch;
    a.T = T; a.K = K; a.R = R;
    a.ktiles = K / kTileK;
    const GemmPlan p = plan_gemm(T, K, R);
    a.ktiles_per_split = p.ktiles_per_split;
    a.xcd_gx = p.xcd ? p.gx : 0;
    if (p.kwave) {
        const size_t lds = (size_t)4 * (32 * slab_pitch<kTileK>() + kTileK) * sizeof(uint16_t);
        const bool scaled = a.s_in != nullptr;
        auto launch = [&](auto kern) -> hipError_t {
            hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
            if (e != hipSuccess) return e;
            hipLaunchKernelGGL(kern, dim3(p.gx, p.gy), dim3(256), lds, stream, a);
            return hipGetLastError();
        };
#define NQ_KW(D, S) (p.rt == 1 ? launch(gemm_kwave_kernel<D, S, 1>) : p.rt == 2 ? launch(gemm_kwave_kernel<D, S, 2>) : launch(gemm_kwave_kernel<D, S, 4>))
        if (dtype == 0) return scaled ? NQ_KW(0, true) : NQ_KW(0, false);
        return scaled ? NQ_KW(1, true) : NQ_KW(1, false);
#undef NQ_KW
    }
    if (p.tt == 1) return dtype == 0 ? launch_gemm<0, 1, 1, 256>(a, p, stream) : launch_gemm<1, 1, 1, 256>(a, p, stream);
    if (dtype == 0) return p.rt == 2 ? launch_gemm<0, 2, 2, 256>(a, p, stream) : launch_gemm<0, 2, 1, 256>(a, p, stream);
    return p.rt == 2 ? launch_gemm<1, 2, 2, 256>(a, p, stream) : launch_gemm<1, 2, 1, 256>(a, p, stream);
}

// More than kKwaveGroupMaxTokens tokens: one launch of gemm_block_group_kernel.  Two row tiles per wavefront halve the
// LDS reads per MFMA and are taken once that still leaves two workgroups for every CU.
static hipError_t gemm_block_group(int dtype, int count, const void* const* x, const uint32_t* const* tiles,
                                   const void* const* s_in, const void* const* s_out, const void* const* bias,
                                   void* const* y, int T, const int* K, const int* R, hipStream_t stream) {
    const int gy = (T + 63) / 64;
    long wide = 0;
    for (int p = 0; p < count; ++p) wide += (long)((R[p] + 255) / 256) * gy;
    const int rt = wide >= 512 ? 2 : 1;
    // Longest k first: the workgroups that run longest start first, the short ones fill in behind them.
    int order[kGroupMax];
    for (int p = 0; p < count; ++p) order[p] = p;
    for (int i = 1; i < count; ++i)
        for (int j = i; j > 0 && K[order[j]] > K[order[j - 1]]; --j) { const int t = order[j]; order[j] = order[j - 1]; order[j - 1] = t; }
    GemmGroup g;
    g.count = count;
    int blocks = 0;
    for (int p = 0; p < kGroupMax; ++p) {
        const int q = order[p < count ? p : count - 1];
        GemmArgs& a = g.a[p];
        a.x = x[q]; a.tiles = (const uint4*)tiles[q];
        a.s_in = (const uint16_t*)(s_in ? s_in[q] : nullptr); a.s_out = (const uint16_t*)(s_out ? s_out[q] : nullptr);
        a.bias = (const uint16_t*)(bias ? bias[q] : nullptr);
        a.y = y[q]; a.acc = nullptr;
        a.T = T; a.K = K[q]; a.R = R[q];
        a.ktiles = K[q] / kTileK; a.ktiles_per_split = a.ktiles;
        a.xcd_gx = (R[q] + 128 * rt - 1) / (128 * rt);
        g.first[p] = blocks;
        if (p < count) blocks += group_blocks(a.xcd_gx, gy);
    }
    g.first[kGroupMax] = blocks;
    for (int p = count; p < kGroupMax; ++p) g.first[p] = blocks;
    const bool scaled = g.a[0].s_in != nullptr;
    const size_t lds = ((size_t)64 * slab_pitch<kTileK>() + kTileK) * sizeof(uint16_t);
    auto launch = [&](auto kern) -> hipError_t {
        hipLaunchKernelGGL(kern, dim3(blocks), dim3(256), lds, stream, g);
        return hipGetLastError();
    };
#define NQ_BG(D, S) (rt == 1 ? launch(gemm_block_group_kernel<D, 1, S>) : launch(gemm_block_group_kernel<D, 2, S>))
    if (dtype == 0) return scaled ? NQ_BG(0, true) : NQ_BG(0, false);
    return scaled ? NQ_BG(1, true) : NQ_BG(1, false);
#undef NQ_BG
}

// GEMMs of several problems on the same token count in one launch; every problem: K % 256 == 0, R % 32 == 0, and
// either all have input scales or none (checked by the caller).  Up to kKwaveGroupMaxTokens tokens the few-token
// tiles, above them block tiles.
hipError_t gemm_onebit_group(int dtype, int count, const void* const* x, const uint32_t* const* tiles,
                             const void* const* s_in, const void* const* s_out, const void* const* bias, void* const* y,
                             int T, const int* K, const int* R, hipStream_t stream) {
    if (count < 1 || count > kGroupMax) return hipErrorInvalidValue;
    if (T > kKwaveGroupMaxTokens) return gemm_block_group(dtype, count, x, tiles, s_in, s_out, bias, y, T, K, R, stream);
    const int gy = (T + 31) / 32;
    int rt = 4;                                  // widest row blocks that still leave two workgroups per CU
    for (; rt > 1; rt /= 2) {
        long total = 0;
        for (int p = 0; p < count; ++p) total += (long)((R[p] / 32 + rt - 1) / rt) * gy;
        if (total >= 512) break;
    }
    // Longest k first: the workgroups that run longest start first, the short ones fill in behind them.
    int order[kGroupMax];
    for (int p = 0; p < count; ++p) order[p] = p;
    for (int i = 1; i < count; ++i)
        for (int j = i; j > 0 && K[order[j]] > K[order[j - 1]]; --j) { const int t = order[j]; order[j] = order[j - 1]; order[j - 1] = t; }
    GemmGroup g;
    g.count = count;
    int blocks = 0;
    for (int p = 0; p < kGroupMax; ++p) {
        const int q = order[p < count ? p : count - 1];
        GemmArgs& a = g.a[p];
        a.x = x[q]; a.tiles = (const uint4*)tiles[q];
        a.s_in = (const uint16_t*)(s_in ? s_in[q] : nullptr); a.s_out = (const uint16_t*)(s_out ? s_out[q] : nullptr);
        a.bias = (const uint16_t*)(bias ? bias[q] : nullptr);
        a.y = y[q]; a.acc = nullptr;
        a.T = T; a.K = K[q]; a.R = R[q];
        a.ktiles = K[q] / kTileK; a.ktiles_per_split = a.ktiles; a.xcd_gx = 0;
        g.first[p] = blocks;
        if (p < count) blocks += ((R[q] / 32 + rt - 1) / rt) * gy;
    }
    g.first[kGroupMax] = blocks;
    for (int p = count; p < kGroupMax; ++p) g.first[p] = blocks;
    const bool scaled = g.a[0].s_in != nullptr;
    const size_t lds = (size_t)4 * (32 * slab_pitch<kTileK>() + kTileK) * sizeof(uint16_t);
    auto launch = [&](auto kern) -> hipError_t {
        hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return e;
        hipLaunchKernelGGL(kern, dim3(blocks), dim3(256), lds, stream, g);
        return hipGetLastError();
    };
#define NQ_KWG(D, S) (rt == 1 ? launch(gemm_kwave_group_kernel<D, S, 1>) : rt == 2 ? launch(gemm_kwave_group_kernel<D, S, 2>) : launch(gemm_kwave_group_kernel<D, S, 4>))
    if (dtype == 0) return scaled ? NQ_KWG(0, true) : NQ_KWG(0, false);
    return scaled ? NQ_KWG(1, true) : NQ_KWG(1, false);
#undef NQ_KWG
}

int gemm_group_max() { return kGroupMax; }
int gemm_group_max_tokens() { return kKwaveGroupMaxTokens; }

}  // namespace nq
