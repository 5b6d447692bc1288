// Prefill at about 128 to 768 tokens: one persistent launch per GEMM stage of a group of linears.
//
//   C[t, j] = s_out[j] * sum_k (x[t, k] * s_in[k]) * sgn(W[j, k])       (same function as nq_gemm.hip)
//
// Replaces, in function only, the tile scheduling and inner product of the reference's prefill kernel
// (src/nanoquant/kernel/cuda/gemm_kernel.cu:525-549 `matmul`, :843-886 tile choice, :594-640 the reduction of
// stripes that share an output tile).  At 128 tokens a whole decoder layer is 20 us of MFMA time, so what counts is
// how much every byte staged and every sign word decoded is reused, and that no compute unit waits for another:
//
//  * A workgroup (4 wavefronts, two workgroups per compute unit) works on a PANEL of 64 tokens x 256 rows.  The
//    activation slab [64 tokens][256 k] is staged once in LDS for all four wavefronts (32 KiB of L2 traffic per
//    8.4 MFLOP; the few-token tiles of nq_gemm.hip stage 16 KiB per 2.1 MFLOP).  Two slabs in LDS: one barrier per
//    k step.  Two workgroups share a compute unit so that one has MFMAs to issue while the other hands over a
//    partial tile or stores a panel, and so that token counts are covered in blocks of 64.
//  * A wavefront holds 64 tokens x 64 rows (four 32x32 accumulators): every sign fragment decoded in registers
//    feeds two MFMAs and every activation fragment read from LDS feeds two (4 lane operations and half an LDS read
//    per MFMA).
//  * Units of work are (panel, k tile of 256); all units of the launch are numbered in one sequence and workgroup w
//    takes the units [w U / G, (w + 1) U / G): every workgroup gets the same number of MFMAs whatever the shapes
//    (stream-k).  A panel whose k range is cut by such boundaries is finished together by the workgroups whose
//    ranges end inside it: each writes its partial 64 x 256 fp32 tile to a workspace slot and raises a flag, and
//    each adds the others' copies of its share of the output tiles and stores them; the workgroup that holds the
//    panel's last unit only contributes.  Stores and loads of partial tiles are device-coherent; a flag is the
//    number of the launch (derived from a counter of workgroup exits kept in the workspace, so nothing has to be
//    cleared between launches or graph replays); waits are bounded and an expiry is reported in the workspace's
//    status word.  A workgroup raises its own flags before it waits for anybody's, and the hardware starts
//    workgroups in the order of their ids with all of them resident: no cycle of waits can form.
#include "nq_common.h"
#include "nq_kernels.h"
#include "nq_mfma.h"

namespace nq {

constexpr int kPanelThreads = 256;
constexpr int kPanelWaves = kPanelThreads / 64;
constexpr int kPanelTok = 64 * (kPanelWaves / 4);           // tokens of a panel: 64 per four wavefronts
constexpr int kPanelRows = 256;                             // rows of a panel
constexpr int kPanelBufHalves = kPanelTok * kTileK + kTileK;   // one slab [tokens][256 k] and its 256 input scales
constexpr int kPanelStagePitch = 40;                        // 16-bit elements per token row of an epilogue staging tile
constexpr int kPanelStageHalves = 32 * kPanelStagePitch;    // per wavefront: one 32 x 32 output tile on its way out
constexpr size_t kPanelLdsBytes = (2 * (size_t)kPanelBufHalves + kPanelWaves * (size_t)kPanelStageHalves) * sizeof(uint16_t);
constexpr int kPanelMax = 16;                               // problems per launch
constexpr int kPanelPerCu = 2;                              // workgroups per compute unit: one computes while the other hands over
constexpr int kPanelSlotFloats = kPanelTok * kPanelRows;    // one partial tile: 64 KiB
constexpr int kPanelFlagStride = 16;                        // uint32 per flag (64 bytes: one flag per cache line)
constexpr size_t kPanelHeadBytes = 256;                     // exit counter (u64 at 0), status word (u32 at 64)

struct PanelProblem {
    const void* x;          // [T, K] 16-bit
    const uint4* tiles;     // [R/32][K/256][64 lanes] 16 bytes each
    const uint16_t* s_in;   // [K] or null
    const uint16_t* s_out;  // [R] or null
    const uint16_t* bias;   // [R] or null
    void* y;                // [T, R] 16-bit
    int K, R, ktiles;
    int first_unit;         // number of the problem's first unit; unused entries: the launch's unit count
};

struct PanelArgs {
    PanelProblem p[kPanelMax];
    int T, tblocks, total_units;
    unsigned spin_limit;
    float* partials;                 // [2 G][kPanelSlotFloats]: slot 2 w for the first segment of workgroup w, 2 w + 1 for its last
    unsigned* flags;                 // [2 G][kPanelFlagStride]
    unsigned long long* exit_count;  // workgroup exits of all launches on this workspace
    unsigned* status;
};

// What a wavefront needs to issue the eight loads of its share of a slab.
struct SlabFetch {
    __amdgpu_buffer_rsrc_t rs;
    uint32_t voff, pass_bytes;
    uint16_t* base;
};

template <int DT, bool SCALED>
// (second argument: wavefronts per SIMD, so that kPanelPerCu workgroups of four wavefronts fit a compute unit)
__global__ __launch_bounds__(kPanelThreads, kPanelPerCu * kPanelWaves / 4) void gemm_panel_kernel(PanelArgs g) {
    using E = Elem<DT>;
    extern __shared__ __attribute__((aligned(16))) uint16_t panel_lds[];
    __shared__ unsigned s_gen;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int th = wave >> 2, rq = wave & 3;                 // token half and row quarter of this wavefront
    // Workgroups go to the 8 XCDs round-robin by their id.  The unit ranges are dealt by a logical index that runs
    // through the workgroups of one XCD first, so that the workgroups of an XCD walk neighbouring panels of the same
    // problems at the same time and find each other's activation slabs in their L2.  (Any bijection is correct; this
    // one is the fast one.)
    const int G = (int)gridDim.x;
    const int wg = (G % 8 == 0) ? ((int)blockIdx.x & 7) * (G >> 3) + ((int)blockIdx.x >> 3) : (int)blockIdx.x;
    const long long U = g.total_units;
    int u = (int)((long long)wg * U / G);
    const int u_end = (int)((long long)(wg + 1) * U / G);

    if (u < u_end) {
        if (tid == 0)
            s_gen = (unsigned)(__hip_atomic_load(g.exit_count, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) / (unsigned long long)G) + 1u;

        // unit u -> problem p, row block rb, token block tb, k tile kt (k tiles run fastest, then token blocks)
        int p = 0;
#pragma unroll
        for (int i = 1; i < kPanelMax; ++i) p += u >= g.p[i].first_unit ? 1 : 0;
        int rb, tb, kt;
        {
            const int local = u - g.p[p].first_unit, kts = g.p[p].ktiles;
            const int per_rb = g.tblocks * kts;
            rb = local / per_rb;
            const int rem = local - rb * per_rb;
            tb = rem / kts;
            kt = rem - tb * kts;
        }

        int p1 = p, rb1 = rb, tb1 = tb, kt1 = kt;     // unit u + 1 (where there is one)
        // Fetching ahead: when this workgroup's range ends inside a panel that BEGINS in it and ends in the next
        // workgroup (a short k range cut once), that workgroup's partial tile is usually there long before this one
        // gets to the panel.  Its flag is looked at one unit ahead and, if set, the sixteen loads of the tile are issued
        // in front of the last unit's MFMAs instead of behind them.  ahead_slot < 0: not that case.  Only for short
        // ranges: the compiler carries the registers of `ahead` through two copies per unit (about 370 cycles), which a
        // range of more than eight units pays more for than the loads hidden once are worth.
        int ahead_slot = -1;
        if (u_end - u >= 2 && u_end - u <= 8) {
            const int lu = u_end - 1;
            int lp = 0;
#pragma unroll
            for (int i = 1; i < kPanelMax; ++i) lp += lu >= g.p[i].first_unit ? 1 : 0;
            const int lkts = g.p[lp].ktiles;
            const int lkt = (lu - g.p[lp].first_unit) % lkts;
            const long long lfirst = (long long)lu - lkt;
            const int next = wg + 1;
            if (lfirst >= u && lkt + 1 < lkts && next < G && (long long)next * U / G != (long long)(next + 1) * U / G &&
                (int)(((lfirst + lkts) * G - 1) / U) == next)
                ahead_slot = 2 * next;
        }
        unsigned ahead_flag = 0;
        bool ahead_loaded = false;
        u32x4_t ahead[8];             // the pieces of the tiles with r = 0; those with r = 1 follow behind the MFMAs
        float16_t acc[2][2];
        auto zero_acc = [&]() {
#pragma unroll
            for (int r = 0; r < 2; ++r)
#pragma unroll
                for (int tt = 0; tt < 2; ++tt)
#pragma unroll
                    for (int v = 0; v < 16; ++v) acc[r][tt][v] = 0.f;
        };
        zero_acc();

        u32x4_t wn[2];          // the wavefront's two weight tiles of the next unit
        u32x4_t w[2];           // ... and of the current one
        // Slab -> LDS without passing through registers (buffer loads with the LDS bit: lane i of an instruction
        // writes 16 bytes at the instruction's LDS base + 16 i).  One instruction fills two token rows of 512 bytes;
        // wavefront w and pass ps take the token pair 8 ps + w.  The slab has no padding, so the sixteen 16-byte
        // chunks of each 256-byte half row are permuted by the token: chunk c of token t sits at c ^ (t & 15), which
        // makes the fragment reads of 16 consecutive tokens at one k offset hit sixteen different bank groups.  A
        // lane picks its SOURCE chunk accordingly (the LDS side of such a load cannot be chosen per lane).  Tokens
        // beyond T lie past the end of the buffer and fill their rows with zeros.
        const int hi = lane >> 5;
        auto slab_fetch_setup = [&](uint16_t* dst, int fp, int ftb, int fkt, bool live) {
            const PanelProblem& P = g.p[fp];
            const uint32_t row_bytes = (uint32_t)P.K * 2u;
            SlabFetch f;
            f.rs = gemm_buffer(P.x, (uint32_t)g.T * row_bytes);
            const int tk0 = 2 * wave + hi;                                  // token of this lane in pass 0
            f.voff = live ? (uint32_t)(ftb * kPanelTok + tk0) * row_bytes + (uint32_t)fkt * (kTileK * 2u) +
                                (uint32_t)(((lane & 31) ^ (tk0 & 15)) * 16)
                          : 0xFFFFFFF0u;
            f.pass_bytes = (uint32_t)(2 * kPanelWaves) * row_bytes;
            f.base = dst + wave * (2 * kTileK);
            if constexpr (SCALED) {
                if (tid < 32 && live) {
                    const __amdgpu_buffer_rsrc_t rss = gemm_buffer(P.s_in, (uint32_t)P.K * 2u);
                    __builtin_amdgcn_raw_ptr_buffer_load_lds(rss, (__attribute__((address_space(3))) void*)(dst + kPanelTok * kTileK),
                                                             16, (uint32_t)fkt * (kTileK * 2u) + (uint32_t)lane * 16u, 0, 0, kGemmCacheDefault);
                }
            }
            return f;
        };
        // pass ps (0..7) of a slab: the two token rows 2 W ps + 2 w, + 1 of wavefront w (W wavefronts).  With four
        // wavefronts a pass is 8 tokens, so bit 3 of the token, which is part of the chunk permutation, alternates
        // with the pass: odd passes take the source chunk with bit 3 flipped (128 bytes further or nearer).
        auto slab_fetch_pass = [&](const SlabFetch& f, int ps) {
            const uint32_t voff = (2 * kPanelWaves * ps) & 8 ? f.voff ^ 128u : f.voff;
            __builtin_amdgcn_raw_ptr_buffer_load_lds(f.rs, (__attribute__((address_space(3))) void*)(f.base + ps * (2 * kPanelWaves * kTileK)), 16,
                                                     voff, (uint32_t)ps * f.pass_bytes, 0, kGemmCacheDefault);
        };
        auto fetch_w = [&](int fp, int frb, int fkt, bool live) {
            const PanelProblem& P = g.p[fp];
            // row tiles beyond R / 32 lie past the end of the buffer and read zeros
            const __amdgpu_buffer_rsrc_t rs = gemm_buffer(P.tiles, (uint32_t)((size_t)(P.R / 32) * P.ktiles * 1024u));
            const int rt = frb * 8 + rq * 2;
#pragma unroll
            for (int r = 0; r < 2; ++r) {
                const uint32_t off = ((uint32_t)(rt + r) * (uint32_t)P.ktiles + (uint32_t)fkt) * 1024u + (uint32_t)lane * 16u;
                wn[r] = __builtin_amdgcn_raw_buffer_load_b128(rs, live ? off : 0xFFFFFFF0u, 0, kGemmCacheDefault);
            }
        };
        // the unit after (p, rb, tb, kt): k tiles run fastest, then token blocks, row blocks, problems
        auto advance = [&](int& ap, int& arb, int& atb, int& akt) {
            if (++akt < g.p[ap].ktiles) return;
            akt = 0;
            if (++atb < g.tblocks) return;
            atb = 0;
            if (++arb * kPanelRows < g.p[ap].R) return;
            arb = 0;
            ++ap;
        };
        if (u + 1 < u_end) advance(p1, rb1, tb1, kt1);
        // The MFMAs of one unit; with `fetch_next` the loads of the next unit's slab and weight tiles are issued
        // between the first k steps, one instruction per step, so that no wavefront queues behind a burst of loads.
        auto compute = [&](const uint16_t* slab, const u32x4_t (&w)[2], bool fetch_next, const SlabFetch& nf) {
            const uint16_t* sc = slab + kPanelTok * kTileK + 8 * hi;
            // token 64 th + 32 tt + (lane & 31): its 16-byte chunk 2 t + hi of the k tile sits at (2 t + hi) ^ (lane & 15)
            const uint16_t* arow = slab + (th * 64 + (lane & 31)) * kTileK;
            const int sw = (lane & 15) ^ hi;
            // (1.0, 1.0) kept in a vector register that the compiler cannot fold: (shifted & mask) | one is then a
            // single and-or instruction (with both as literals it is an AND and an OR)
            uint32_t one = E::kOnePair;
            asm volatile("" : "+v"(one));
            // The activation fragments of step t + 1 are read from LDS before the MFMAs of step t are issued (the
            // scheduling barrier keeps the compiler from moving the reads back in front of their use).
            auto read_a = [&](int t, uint4 (&a)[2]) {
                const uint16_t* ap = arow + 128 * (t >> 3) + (((2 * (t & 7)) ^ sw) << 3);
                a[0] = *(const uint4*)(ap);
                a[1] = *(const uint4*)(ap + 32 * kTileK);
            };
            uint4 a_now[2], a_next[2];
            read_a(0, a_now);
#pragma unroll
            for (int t = 0; t < 16; ++t) {
                const int s = 4 * (t & 3);
                // no branch inside the k steps: without a next unit the same loads are issued past the end of their
                // buffers (they move nothing)
                if (t == 0) fetch_w(p1, rb1, kt1, fetch_next);
                if (t >= 1 && t <= 8) slab_fetch_pass(nf, t - 1);
                uint4 sp;
                if constexpr (SCALED) sp = *(const uint4*)(sc + 16 * t);   // broadcast read
                if (t + 1 < 16) read_a(t + 1, a_next);
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int r = 0; r < 2; ++r) {
                    const uint32_t word = w[r][t >> 2];
                    uint4 b;
                    if constexpr (SCALED) {
                        // +-s_in[k]: the scale pair with its sign bits flipped by the packed bits, so that
                        // x * s_in is formed exactly inside the MFMA
                        b.x = sp.x ^ ((word << (s + 0)) & kSignPair);
                        b.y = sp.y ^ ((word << (s + 1)) & kSignPair);
                        b.z = sp.z ^ ((word << (s + 2)) & kSignPair);
                        b.w = sp.w ^ ((word << (s + 3)) & kSignPair);
                    } else {
                        b.x = ((word << (s + 0)) & kSignPair) | one;
                        b.y = ((word << (s + 1)) & kSignPair) | one;
                        b.z = ((word << (s + 2)) & kSignPair) | one;
                        b.w = ((word << (s + 3)) & kSignPair) | one;
                    }
                    acc[r][0] = Mfma<DT>::run(a_now[0], b, acc[r][0]);
                    acc[r][1] = Mfma<DT>::run(a_now[1], b, acc[r][1]);
                }
                a_now[0] = a_next[0]; a_now[1] = a_next[1];
            }
        };
        // Accumulator element v of lane l of tile (r, tt): token 64 th + 32 tt + 8 (v >> 2) + 4 (l >> 5) + (v & 3),
        // row 32 (8 rb + 2 rq + r) + (l & 31).  A tile is scaled, converted and turned round in the wavefront's
        // staging area (rows of one token next to each other), then leaves as 16-byte stores: lane l stores rows
        // 8 (l & 3) .. + 7 of token (l >> 2) and of token 16 + (l >> 2).  With all four tiles in `tile_mask` always 8
        // store instructions per wavefront: tokens beyond T and row tiles beyond R are pointed past the end of the
        // buffer and dropped.
        auto epilogue = [&](int ep, int erb, int etb, unsigned tile_mask) {
            const PanelProblem& P = g.p[ep];
            uint16_t* stage = panel_lds + 2 * kPanelBufHalves + wave * kPanelStageHalves;
            const uint32_t row_bytes = (uint32_t)P.R * 2u;
            const __amdgpu_buffer_rsrc_t ry = gemm_buffer(P.y, (uint32_t)g.T * row_bytes);
#pragma unroll
            for (int r = 0; r < 2; ++r) {
                const int row0 = (erb * 8 + rq * 2 + r) * 32;
                const bool live = row0 < P.R;             // whole tiles only: uniform over the wavefront
                float sc = 1.f, bs = 0.f;
                if (live && P.s_out) sc = E::to_float(P.s_out[row0 + (lane & 31)]);
                if (live && P.bias) bs = E::to_float(P.bias[row0 + (lane & 31)]);
#pragma unroll
                for (int tt = 0; tt < 2; ++tt) {
                    if (!((tile_mask >> (2 * r + tt)) & 1u)) continue;        // finished by another workgroup
#pragma unroll
                    for (int v = 0; v < 16; ++v)
                        stage[(8 * (v >> 2) + 4 * hi + (v & 3)) * kPanelStagePitch + (lane & 31)] = E::from_float_sat(acc[r][tt][v] * sc + bs);
                    const int tok0 = etb * kPanelTok + th * 64 + tt * 32 + (lane >> 2);
#pragma unroll
                    for (int half = 0; half < 2; ++half) {
                        const u32x4_t out = *(const u32x4_t*)(stage + ((lane >> 2) + 16 * half) * kPanelStagePitch + 8 * (lane & 3));
                        const uint32_t off = live ? (uint32_t)(tok0 + 16 * half) * row_bytes + (uint32_t)(row0 + 8 * (lane & 3)) * 2u : 0xFFFFFFF0u;
                        __builtin_amdgcn_raw_buffer_store_b128(out, ry, off, 0, kGemmCacheDefault);
                    }
                }
            }
        };
        // A partial tile in its slot: 16-byte piece i = 8 r + 4 tt + (v >> 2) of wavefront w and lane l at
        // ((16 w + i) * 64 + l) * 16 bytes, so every store and load instruction moves one contiguous KiB.
        auto partial_rsrc = [&](int slot) {
            return gemm_buffer(g.partials + (size_t)slot * kPanelSlotFloats, (uint32_t)(kPanelSlotFloats * sizeof(float)));
        };
        auto write_partial = [&](int slot) {
            const __amdgpu_buffer_rsrc_t rs = partial_rsrc(slot);
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                const int r = i >> 3, tt = (i >> 2) & 1, j = i & 3;
                u32x4_t v;
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const float f = acc[r][tt][4 * j + e];
                    v[e] = __builtin_bit_cast(uint32_t, f);
                }
                __builtin_amdgcn_raw_buffer_store_b128(v, rs, (uint32_t)lane * 16u, (uint32_t)(wave * 16 + i) * 1024u, kGemmCacheAgent);
            }
        };
        // adds tile q = 2 r + tt (four 16-byte pieces per lane) of the partial tiles in slots sa and sb to this
        // wavefront's accumulators; both sets of loads are in flight together (sb < 0: only sa)
        auto add_partial_tile = [&](int q, int sa, int sb) {
            const __amdgpu_buffer_rsrc_t ra = partial_rsrc(sa);
            const __amdgpu_buffer_rsrc_t rb_ = partial_rsrc(sb < 0 ? sa : sb);
            const uint32_t off_b = sb < 0 ? 0xFFFFFFF0u : (uint32_t)lane * 16u;     // past the end: reads zeros
            u32x4_t va[4], vb[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                va[j] = __builtin_amdgcn_raw_buffer_load_b128(ra, (uint32_t)lane * 16u, (uint32_t)(wave * 16 + q * 4 + j) * 1024u, kGemmCacheAgent);
                vb[j] = __builtin_amdgcn_raw_buffer_load_b128(rb_, off_b, (uint32_t)(wave * 16 + q * 4 + j) * 1024u, kGemmCacheAgent);
            }
#pragma unroll
            for (int r = 0; r < 2; ++r)
#pragma unroll
                for (int tt = 0; tt < 2; ++tt) {
                    if (2 * r + tt != q) continue;
#pragma unroll
                    for (int j = 0; j < 4; ++j)
#pragma unroll
                        for (int e = 0; e < 4; ++e) {
                            const uint32_t xa = va[j][e], xb = vb[j][e];
                            acc[r][tt][4 * j + e] += __builtin_bit_cast(float, xa) + __builtin_bit_cast(float, xb);
                        }
                }
        };
        // The loads of the next slab write LDS behind the compiler's back; it would make every LDS read that follows
        // them wait for them unless it can see that the two do not overlap.  The __restrict__ parameters say so: the
        // buffer the MFMAs read and the buffer the loads fill are different halves of the LDS allocation.
        auto unit_body = [&](const uint16_t* __restrict__ slab_now, uint16_t* __restrict__ slab_next, bool fetch_next) {
            const SlabFetch nf = slab_fetch_setup(slab_next, p1, tb1, kt1, fetch_next);
            compute(slab_now, w, fetch_next, nf);
        };
        {
            const SlabFetch f0 = slab_fetch_setup(panel_lds, p, tb, kt, true);
#pragma unroll
            for (int ps = 0; ps < 8; ++ps) slab_fetch_pass(f0, ps);
        }
        fetch_w(p, rb, kt, true);
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        w[0] = wn[0]; w[1] = wn[1];
        lds_barrier();
        const unsigned gen = s_gen;
        int cur = 0;
        int seg_kt0 = kt;         // first k tile of the segment (the run of units inside one panel) being summed
        int flag_state = 0;       // 1: partial tile stored in this iteration, 2: stored an iteration ago (flag is due)
#pragma unroll 1
        while (true) {
            const int kts = g.p[p].ktiles;
            const bool more = u + 1 < u_end;
            const bool last_kt = kt + 1 == kts;
            if (ahead_slot >= 0) {
                if (u + 2 == u_end) {
                    if (lane == 0) ahead_flag = __hip_atomic_load(g.flags + (size_t)ahead_slot * kPanelFlagStride, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                } else if (u + 1 == u_end) {
                    if ((unsigned)__builtin_amdgcn_readfirstlane((int)ahead_flag) == gen) {
                        const __amdgpu_buffer_rsrc_t ra = partial_rsrc(ahead_slot);
#pragma unroll
                        for (int i = 0; i < 8; ++i)
                            ahead[i] = __builtin_amdgcn_raw_buffer_load_b128(ra, (uint32_t)lane * 16u, (uint32_t)(wave * 16 + i) * 1024u, kGemmCacheAgent);
                        ahead_loaded = true;
                    }
                }
            }
            unit_body(panel_lds + cur * kPanelBufHalves, panel_lds + (cur ^ 1) * kPanelBufHalves, more);
            int stores = 0;       // store instructions of this wavefront issued behind the loads above
            if (last_kt || !more) {
                if (seg_kt0 == 0 && last_kt) {
                    epilogue(p, rb, tb, 0xFu);            // the whole k range of the panel was this workgroup's
                    stores = 8;
                } else if (last_kt) {
                    // The last k tiles of a panel that began in earlier workgroups (always the first segment of a
                    // range): hand the partial tile over and go on; the flag follows when the stores have arrived.
                    write_partial(2 * wg);
                    flag_state = 1;
                    stores = 16;
                } else {
                    // The range ends inside the panel.  All workgroups in this position (the one with the panel's first
                    // k tile and those that lie wholly inside it) finish the panel TOGETHER: each publishes its partial
                    // tile, waits for everybody's, and sums and stores its share of the 32 output tiles (tile q of
                    // wavefront w belongs to the workgroup with index (4 w + q) mod n among them), so that the time
                    // of the reduction does not grow with the number of workgroups a long k range is shared by.
                    // First raise the flag of this workgroup's earlier partial tile if that is still due: the
                    // workgroups finishing THAT panel must not wait for what follows here.
                    if (flag_state != 0) {
                        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
                        lds_barrier();
                        if (tid == 0) __hip_atomic_store(g.flags + (size_t)(2 * wg) * kPanelFlagStride, gen, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                        flag_state = 0;
                    }
                    auto has_units = [&](int c) { return (long long)c * U / G != (long long)(c + 1) * U / G; };
                    const long long panel_first = (long long)(u - kt);
                    const int w_first = (int)(((panel_first + 1) * G - 1) / U);
                    const int w_last = (int)(((panel_first + kts) * G - 1) / U);      // holds the panel's last unit
                    int n = 0, mine = 0;
                    for (int c = w_first; c < w_last; ++c) {
                        if (!has_units(c)) continue;
                        if (c == wg) mine = n;
                        ++n;
                    }
                    if (n > 1) {
                        write_partial(2 * wg + 1);
                        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
                        lds_barrier();
                        if (tid == 0) __hip_atomic_store(g.flags + (size_t)(2 * wg + 1) * kPanelFlagStride, gen, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    }
                    // everybody else's partial tile: the last workgroup's is the one of its first segment
                    bool ok = true;
#pragma unroll 1
                    for (int c = w_first; c <= w_last && ok; ++c) {
                        if (c == wg || !has_units(c) || ahead_loaded) continue;
                        const unsigned* flag = g.flags + (size_t)(c == w_last ? 2 * c : 2 * c + 1) * kPanelFlagStride;
                        unsigned spins = 0;
                        while (true) {
                            unsigned f = 0;
                            if (lane == 0) f = __hip_atomic_load(flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                            f = (unsigned)__builtin_amdgcn_readfirstlane((int)f);
                            if (f == gen) break;
                            __builtin_amdgcn_s_sleep(4);
                            if (++spins >= g.spin_limit) {           // bounded wait: report, finish with what is there
                                if (lane == 0) atomicOr(g.status, 1u);
                                ok = false;
                                break;
                            }
                        }
                    }
                    unsigned tile_mask = 0;
                    if (n == 1 && ahead_loaded) {
                        const __amdgpu_buffer_rsrc_t rt_ = partial_rsrc(ahead_slot);
                        u32x4_t v[8];
#pragma unroll
                        for (int i = 0; i < 8; ++i)
                            v[i] = __builtin_amdgcn_raw_buffer_load_b128(rt_, (uint32_t)lane * 16u, (uint32_t)(wave * 16 + 8 + i) * 1024u, kGemmCacheAgent);
#pragma unroll
                        for (int i = 0; i < 8; ++i)
#pragma unroll
                            for (int e = 0; e < 4; ++e) {
                                const uint32_t x = ahead[i][e];
                                acc[0][(i >> 2) & 1][4 * (i & 3) + e] += __builtin_bit_cast(float, x);
                            }
#pragma unroll
                        for (int i = 0; i < 8; ++i)
#pragma unroll
                            for (int e = 0; e < 4; ++e) {
                                const uint32_t x = v[i][e];
                                acc[1][(i >> 2) & 1][4 * (i & 3) + e] += __builtin_bit_cast(float, x);
                            }
                        tile_mask = 0xFu;
                    } else if (n == 1 && ok) {
                        // the common case of a short k range: this workgroup and the one behind it.  All four tiles
                        // are this workgroup's, and their sixteen loads go out together.
                        const __amdgpu_buffer_rsrc_t rt_ = partial_rsrc(2 * w_last);
                        u32x4_t v[16];
#pragma unroll
                        for (int i = 0; i < 16; ++i)
                            v[i] = __builtin_amdgcn_raw_buffer_load_b128(rt_, (uint32_t)lane * 16u, (uint32_t)(wave * 16 + i) * 1024u, kGemmCacheAgent);
#pragma unroll
                        for (int i = 0; i < 16; ++i)
#pragma unroll
                            for (int e = 0; e < 4; ++e) {
                                const uint32_t x = v[i][e];
                                acc[i >> 3][(i >> 2) & 1][4 * (i & 3) + e] += __builtin_bit_cast(float, x);
                            }
                        tile_mask = 0xFu;
                    } else
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        if ((wave * 4 + q) % n != mine) continue;
                        tile_mask |= 1u << q;
                        if (!ok) continue;
                        int held = -1;                    // a slot waiting for a partner to be loaded with
#pragma unroll 1
                        for (int c = w_first; c <= w_last; ++c) {
                            if (c == wg || !has_units(c)) continue;
                            const int slot = c == w_last ? 2 * c : 2 * c + 1;
                            if (held < 0) { held = slot; continue; }
                            add_partial_tile(q, held, slot);
                            held = -1;
                        }
                        if (held >= 0) add_partial_tile(q, held, -1);
                    }
                    epilogue(p, rb, tb, tile_mask);
                }
                zero_acc();
                seg_kt0 = 0;
            }
            if (!more) break;
            // The next slab must have landed in LDS before anyone reads it.  The counter of outstanding memory
            // operations runs in issue order, so the stores just issued (which nobody here waits for) may stay in
            // flight; the partial tile stored an iteration ago is complete once the counter has been at zero.
            if (stores == 16) asm volatile("s_waitcnt vmcnt(16)" ::: "memory");
            else if (stores == 8) asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
            else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            w[0] = wn[0]; w[1] = wn[1];
            lds_barrier();
            if (flag_state == 2 && stores == 0) {
                if (tid == 0) __hip_atomic_store(g.flags + (size_t)(2 * wg) * kPanelFlagStride, gen, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                flag_state = 0;
            }
            if (flag_state == 1) flag_state = 2;
            cur ^= 1;
            p = p1; rb = rb1; tb = tb1; kt = kt1;
            ++u;
            if (u + 1 < u_end) advance(p1, rb1, tb1, kt1);
        }
        if (flag_state != 0) {
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            lds_barrier();
            if (tid == 0) __hip_atomic_store(g.flags + (size_t)(2 * wg) * kPanelFlagStride, gen, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    }
    if (tid == 0) __hip_atomic_fetch_add(g.exit_count, 1ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// ---- host side --------------------------------------------------------------------------------
// Workgroups of a launch: kPanelPerCu per compute unit, all resident at once (checked against the occupancy of the
// kernel before the first launch on a device).
static int panel_grid() {
    static PerDeviceFlag known;
    static int cus[64];
    const int dev = current_device();
    if (dev >= 0 && dev < 64 && known.test(dev)) return cus[dev];
    int n = 0;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev < 0 ? 0 : dev) != hipSuccess || n <= 0) return 0;
    n *= kPanelPerCu;
    if (dev >= 0 && dev < 64) { cus[dev] = n; known.set(dev); }
    return n;
}

size_t panel_workspace_bytes() {
    const int G = panel_grid();
    if (G <= 0) return 0;
    const size_t flags = ((size_t)2 * G * kPanelFlagStride * sizeof(unsigned) + 255) / 256 * 256;
    return kPanelHeadBytes + flags + (size_t)2 * G * kPanelSlotFloats * sizeof(float);
}

// Whether one stage of a group is better off as a panel launch than on the tiles of nq_gemm.hip (measured on
// Llama-2-7B layers, per stage, 64 .. 4096 tokens).  Every workgroup must get a few k steps (otherwise panels are cut
// into many pieces and the hand-over of partial tiles costs more than the shared slabs save); the longest k range
// must not be shared by too many workgroups (the first stage of a 128-token layer, whose 43-tile down projection is
// cut eight ways, is faster on the few-token tiles); token counts that fill their 64-token blocks badly waste MFMAs,
// which only a stage with a long k makes up for (its block tiles need a k split and a finish launch); and from
// about 1024 tokens on the block tiles are level.
bool panel_applies(int count, int T, const int* K, const int* R) {
    const int G = panel_grid();
    if (G <= 0 || count < 1 || count > kPanelMax || T < 1 || T > 768) return false;
    const int tblocks = (T + kPanelTok - 1) / kPanelTok;
    long long units = 0;
    int longest = 0;
    for (int p = 0; p < count; ++p) {
        if (K[p] % kTileK != 0 || R[p] % 32 != 0) return false;
        units += (long long)((R[p] + kPanelRows - 1) / kPanelRows) * tblocks * (K[p] / kTileK);
        longest = longest > K[p] / kTileK ? longest : K[p] / kTileK;
    }
    const double per_wg = (double)units / G;
    if (per_wg < 3.0) return false;
    // up to two token blocks the few-token tiles are the alternative, and a strong one; beyond, panels win more easily
    const bool few = T <= 2 * kPanelTok;
    if (longest > (few ? 4.0 : 8.0) * per_wg) return false;
    const double fill = (double)T / (tblocks * kPanelTok);
    return fill >= (few ? 0.78 : 0.70) || longest > 16;
}

template <int DT, bool SCALED>
static hipError_t launch_panel(const PanelArgs& a, int G, hipStream_t stream) {
    auto kern = gemm_panel_kernel<DT, SCALED>;
    static PerDeviceFlag attr_done;
    const int dev = current_device();
    if (!attr_done.test(dev)) {
        hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)kPanelLdsBytes);
        if (e != hipSuccess) return e;
        int per_cu = 0;
        e = hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, (const void*)kern, kPanelThreads, kPanelLdsBytes);
        if (e != hipSuccess) return e;
        if (per_cu < kPanelPerCu) return hipErrorLaunchOutOfResources;
        attr_done.set(dev);
    }
    hipLaunchKernelGGL(kern, dim3(G), dim3(kPanelThreads), kPanelLdsBytes, stream, a);
    return hipGetLastError();
}

// One launch for the GEMMs of `count` problems on the same T tokens (s_in: all or none).  `workspace`:
// panel_workspace_bytes() bytes, zero when first used and owned by these launches from then on.
hipError_t gemm_panel_group(int dtype, int count, const void* const* x, const uint32_t* const* tiles,
                            const void* const* s_in, const void* const* s_out, const void* const* bias, void* const* y,
                            int T, const int* K, const int* R, void* workspace, unsigned spin_limit, hipStream_t stream) {
    const int G = panel_grid();
    if (G <= 0) return hipErrorInvalidDevice;
    if (count < 1 || count > kPanelMax || T < 1 || !workspace) return hipErrorInvalidValue;
    PanelArgs a;
    a.T = T;
    a.tblocks = (T + kPanelTok - 1) / kPanelTok;
    long long units = 0;
    for (int p = 0; p < kPanelMax; ++p) {
        const int q = p < count ? p : count - 1;
        PanelProblem& P = a.p[p];
        P.x = x[q]; P.tiles = (const uint4*)tiles[q];
        P.s_in = (const uint16_t*)(s_in ? s_in[q] : nullptr);
        P.s_out = (const uint16_t*)(s_out ? s_out[q] : nullptr);
        P.bias = (const uint16_t*)(bias ? bias[q] : nullptr);
        P.y = y[q];
        P.K = K[q]; P.R = R[q]; P.ktiles = K[q] / kTileK;
        P.first_unit = (int)units;
        if (p < count) units += (long long)((R[q] + kPanelRows - 1) / kPanelRows) * a.tblocks * P.ktiles;
        if (units > 0x7FFFFFFF) return hipErrorInvalidValue;
    }
    a.total_units = (int)units;
    a.spin_limit = spin_limit ? spin_limit : (1u << 20);
    char* base = (char*)workspace;
    const size_t flags = ((size_t)2 * G * kPanelFlagStride * sizeof(unsigned) + 255) / 256 * 256;
    a.exit_count = (unsigned long long*)base;
    a.status = (unsigned*)(base + 64);
    a.flags = (unsigned*)(base + kPanelHeadBytes);
    a.partials = (float*)(base + kPanelHeadBytes + flags);
    const bool scaled = a.p[0].s_in != nullptr;
    if (dtype == 0) return scaled ? launch_panel<0, true>(a, G, stream) : launch_panel<0, false>(a, G, stream);
    return scaled ? launch_panel<1, true>(a, G, stream) : launch_panel<1, false>(a, G, stream);
}

}  // namespace nq
