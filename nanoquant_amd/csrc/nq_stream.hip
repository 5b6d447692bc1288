// Decode path, run-list form: ONE launch covers a whole list of stages (out[b, row] = s_row[row] * sum of
// signed, scaled inputs; two stages per linear).
//
// A decoder stack at batch 1 is a stream of small sign matrices (1-6 MB each) and a 4096x4096 layer
// is worth 0.3 us of HBM time, so launching one kernel per stage (as the reference does,
// src/nanoquant/kernel/cuda/gemv_kernel.cu:406-425: two launches per linear) leaves the memory system
// idle most of the time.  Here the grid is exactly as large as the device can keep resident (one 1024-lane
// workgroup per CU) and the stages are grouped into phases by dependency depth (all first stages of
// independent linears are phase 0, their second stages phase 1, ...):
//   * every workgroup owns a balanced slice (in units of sign words) of every phase, cut at row
//     boundaries by the host: no workgroup slot ever idles while another phase is running;
//   * a slice whose input is produced by an earlier stage waits on that stage's completion counters
//     (device-scope atomics), not on a kernel boundary.  All workgroups are resident, so the producers
//     are always running; the wait is bounded all the same and an expiry is reported through the
//     status word;
//   * the intermediate h is handed over with relaxed device-scope atomics (coherent 32/64-bit
//     accesses) instead of cache-wide release/acquire fences, which on this part write back and
//     invalidate a whole L2 per workgroup;
//   * inside a workgroup the sign words go to the MFMA units as (16 rows x 4 units) items, one row and unit
//     per lane; wavefronts take contiguous runs of items and finish per-row sums with LDS float atomics.
// The arithmetic per 16-byte unit is in nq_decode.h.
#include <type_traits>

#include "nq_decode.h"
#include "nq_kernels.h"

namespace nq {

// fp4 x fp8 arithmetic: rows whose sums a workgroup keeps in LDS at a time (then: barrier, scale, store, barrier).
// Every block of a slice ends with all wavefronts waiting for the slowest one, so few large blocks: 1024 rows (16 KiB
// of row sums at batch 4; 256-row blocks cost the batch-4 stack 8.6 instead of 6.2 us per layer).  The 16-bit
// arithmetic (batch 8 and 16) keeps its row sums in registers and has no row blocks.
__host__ __device__ constexpr int row_block(int batch) { return batch <= 8 ? 1024 : 256; }
// Same-address device-scope atomics serialise at the memory side (tens of ns each), so completion
// counts are spread over kSubCounters addresses per stage and kExitSubs addresses for the exit count,
// one 64-byte line each.
constexpr int kSubCounters = 8;
constexpr int kExitSubs = 64;
constexpr int kCounterStride = 8;              // 64-bit words between sub-counters
// Counters are 64-bit and only ever grow: launch number g of a run list finds every exit sub-counter k
// in [g*members_k, (g+1)*members_k) for as long as the reading workgroup itself has not left, so
// g = value / members_k needs no reset between launches and no atomic that returns a value; stage s
// is complete in launch g when its sub-counters add up to (g+1) * seg_count(s).
constexpr size_t kStreamShareBytes = 15 * 1024; // column shares of the 16-bit arithmetic: (1024 / 64 - 1) wavefronts x 64 lanes x 16 bytes
constexpr int kQ8Depth = 3;                    // items (2 KB of packed words each) in flight per wavefront, fp4 x fp8 path
constexpr int kStreamLdsMax = 160 * 1024 - 512;   // staged activations + row accumulators: the LDS of a CU less the static variables

// The packed words of one stage as a raw buffer: one 16-byte load per unit whatever the row alignment
// (buffer loads need dword alignment only), zeros past the end of the matrix, and "no load" expressed
// as an offset past the end instead of a branch -- with exactly one load instruction per loop trip the
// compiler can leave younger fetches in flight (vmcnt counting) instead of waiting for all of them.
// Cache policy of the packed-word fetches: default.  The non-temporal hint costs a fifth of the read bandwidth here
// (a wave-load is 16 rows x 64 bytes, so every 128-byte line is asked for twice, and the hint drops it in between).
#ifndef NQ_BITS_AUX
#define NQ_BITS_AUX 0
#endif
struct BitsView {
    __amdgpu_buffer_rsrc_t rsrc;
    int words;      // 32-bit words per row
    int ragged;     // row-major and words % 4 != 0: the last unit of a row holds fewer than 4 words
    int groups;     // > 0: tile order (see tile_kernel), value = 4-unit groups per row; 0: row-major
};

__device__ __forceinline__ BitsView bits_view(const RunStage& st) {
    BitsView v;
    v.words = st.words;
    v.groups = st.tiled ? (st.words + 15) >> 4 : 0;
    const size_t bytes = st.tiled ? (size_t)((st.rows + 31) >> 5) * v.groups * 2048 : (size_t)st.rows * st.words * sizeof(uint32_t);
    v.rsrc = raw_buffer(st.bits, (uint32_t)bytes);
    v.ragged = !st.tiled && (st.words & 3) != 0;
    return v;
}

// In tile order the 64 units of a wave-load (16 rows x 4 units) are 1 KiB contiguous and every line is read once:
// streamed with the non-temporal hint (6.5 TB/s in a read-only probe against 5.9 row-major with default policy).
// ORDER: 0 = as the view says (a branch, two load instructions), 1 = tile order, 2 = row-major: a loop that keeps several
// fetches in flight wants exactly one load instruction per fetch, or the compiler waits for all of them at every use.
template <int ORDER = 0>
__device__ __forceinline__ uint4 load_unit(const BitsView& v, int row, int unit, bool live) {
    u32x4_t w;
    if (ORDER == 1 || (ORDER == 0 && v.groups)) {
        const uint32_t r = (uint32_t)row, u = (uint32_t)unit;
        const uint32_t idx = ((((r >> 5) * (uint32_t)v.groups + (u >> 2)) * 2u + ((r >> 4) & 1u)) * 4u + (u & 3u)) * 16u + (r & 15u);
        w = __builtin_amdgcn_raw_buffer_load_b128(v.rsrc, live ? idx * 16u : kPastEnd, 0, 2 /* nt */);
    } else {
        const uint32_t off = live ? ((uint32_t)row * (uint32_t)v.words + 4u * (uint32_t)unit) * 4u : kPastEnd;
        w = __builtin_amdgcn_raw_buffer_load_b128(v.rsrc, off, 0, NQ_BITS_AUX);
    }
    return make_uint4(w.x, w.y, w.z, w.w);
}

// To be applied where a fetched unit is consumed (not where it is fetched: that would wait for the load):
// the last unit of a ragged row holds fewer than 4 words of it, the rest belong to the next row.
__device__ __forceinline__ void trim_unit(const BitsView& v, uint4& w, int unit) {
    if (v.ragged) {
        const int left = v.words - 4 * unit;
        if (left < 4) w.w = 0;
        if (left < 3) w.z = 0;
        if (left < 2) w.y = 0;
    }
}

// Bytes of LDS in front of the staged input: row sums and two sets of input totals [2][16].  Reproducible sums (det):
// a second set of row sums (what earlier input chunks of the row block added up to), two sets of per-wavefront input
// totals [2][16][4] and two exponent words.
// The 16-bit arithmetic keeps its row sums in registers; its LDS head holds the totals of the staged units
// ([batch][units + 1] floats, added up in unit order: no LDS atomics, so the results do not depend on their order).
constexpr int kUnitTotalsBytes = 4096;
// own: the fp4 x fp8 variant whose wavefronts own row pairs keeps no row sums in LDS.
__host__ __device__ constexpr size_t stream_head_bytes(int batch, int arith, bool det = false, bool own = false) {
    return arith == 2 ? (own ? 0 : (size_t)row_block(batch) * batch * sizeof(float) * (det ? 2 : 1)) + (det ? 1024 : 128)
                      : (size_t)kUnitTotalsBytes + 128;
}

// fp4 x fp8 arithmetic: items that each wavefront of a workgroup takes (contiguous runs).
__host__ __device__ __forceinline__ int mfma_items_per_wave(int nitems, int waves) { return (nitems + waves - 1) / waves; }

// ARITH: 1 = MFMA with 16-bit operands, 2 = MFMA with one-bit fp4 weights and fp8 pieces of the input (batch <= 4).
// DET, fp4 x fp8 arithmetic: row sums that do not depend on the order in which the wavefronts of a workgroup add
// their partial sums.  Every partial sum is rounded to a grid fine enough (2^-22 of columns x largest staged value, a
// bound on every sum of the chunk) that all additions into a row sum are exact; the input totals are kept per wavefront
// and added in wavefront order; the row sums of successive input chunks (different grids) are added one chunk after
// the other.  Costs up to 16 bits below that bound in precision, two barriers per chunk of a long input, 4 KiB of LDS.
// TILED (fp4 x fp8 arithmetic only): every stage of the list has its words in tile order; the 16-bit arithmetic reads
// either order, stage by stage.
// OWN (fp4 x fp8 arithmetic in tile order, every input staged in one chunk): a wavefront owns whole row pairs (32 rows)
// of a slice and walks all their columns, so the row sums stay in its MFMA accumulators and go from there to the output:
// no row sums in LDS, no LDS atomics, no barrier and no epilogue pass per row block.  The first pair of wavefront w is
// pair w; every further one comes from a counter in LDS, so a wavefront that is served faster takes more pairs (the
// four wavefronts of a SIMD are served oldest first; with equal shares the oldest waits 40 % of every pass).
template <int DT, int BATCH, int ARITH, int THREADS, bool SINGLE, bool TILED, bool DET = false, bool OWN = false>
__global__ __launch_bounds__(THREADS) void gemv_stream_kernel(int nstages, const RunSlice* __restrict__ slices,
                                                                     unsigned long long* counters, unsigned* status,
                                                                     unsigned spin_limit, int chunk_cap,
                                                                     RunStage single, int single_rows,
                                                                     const void* ext_in, void* ext_out) {
    using E = Elem<DT>;
    constexpr int kStreamThreads = THREADS;
    constexpr int kWaves = THREADS / kWave;
    constexpr int kRowBlock = row_block(BATCH);
    extern __shared__ uint4 lds_raw[];
    static_assert(ARITH == 1 || ARITH == 2, "unknown arithmetic");
    constexpr bool kQ8 = ARITH == 2;
    static_assert(!OWN || (kQ8 && TILED && !SINGLE), "owned row pairs exist for the tile-order fp4 x fp8 kernel only");
    constexpr bool kTotals = true;                              // both arithmetics: signed sum = (sum of x) - 2 (sum of b x)
    static_assert(!kQ8 || BATCH * kQ8Pieces <= 16, "pieces of all batch rows must fit the 16 operand columns");
    constexpr int kRaccFloats = kQ8 ? (OWN ? 0 : kRowBlock * BATCH) : kUnitTotalsBytes / (int)sizeof(float);   // 16-bit arithmetic: the unit totals
    float* racc = (float*)lds_raw;                              // [kRowBlock][BATCH] row sums
    float* rtot = racc + kRaccFloats;                           // DET: the same, summed over the input chunks done so far
    // [2][16] sum of the staged input per batch row (DET: [2][16 wavefronts][4]); slices alternate between the two, so
    // that the one of the next slice is cleared a barrier ahead of its staging instead of costing a barrier of its own
    constexpr int kTotStride = (DET && kQ8) ? 64 : 16;
    float* xtot_base = racc + kRaccFloats * (DET && kQ8 ? 2 : 1);
    uint32_t* ebmax_base = (uint32_t*)(xtot_base + 2 * kTotStride);   // DET: [2] largest unit exponent of the staged input
    uint4* xs_base = lds_raw + stream_head_bytes(BATCH, ARITH, DET, OWN) / sizeof(uint4);
    __shared__ int s_flag;
    __shared__ int s_pair;                                      // OWN: the next row pair of the slice that nobody has taken
    const int tid = threadIdx.x;
    const int wg = blockIdx.x;
    if (tid == 0) s_flag = 0;
    if (tid < 2 * kTotStride) xtot_base[tid] = 0.f;
    if (DET && kQ8 && tid < 2) ebmax_base[tid] = 0u;
    int slice_count = 0;

    // Which launch of this run list is this?  Needed only by waiting slices; the load is issued now and
    // its latency is hidden behind phase 0.
    unsigned long long gen_raw = 0;
    unsigned members = 1;
    if (tid < kWave && !SINGLE) {
        const unsigned long long* exit_sub = counters + (size_t)nstages * kSubCounters * kCounterStride;
        const unsigned total = gridDim.x;
        const unsigned sub = (unsigned)wg & (kExitSubs - 1);
        members = (total + kExitSubs - 1 - sub) / kExitSubs;
        gen_raw = __hip_atomic_load(exit_sub + (size_t)sub * kCounterStride, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    bool aborted = false;

    // fp4 x fp8 arithmetic: the three item fetches (2 KB of packed words each) that a wavefront keeps in flight.  In
    // tile order they run on across passes and slices: while a wavefront works off the last items of a pass, its
    // refills already ask for the first items of the next pass (next input chunk, next row block or next slice --
    // packed words depend on nothing), so the stream does not stop for the epilogue, the dependency wait and the
    // staging in between.  A pass is walked in P = 3 ceil(max(items, 3) / 3) positions (positions past the last
    // item only refill), so the rotation of the three register pairs starts every pass at pair 0.
    const int qlane = tid & 63;
    const int qwave = __builtin_amdgcn_readfirstlane(tid >> 6);                   // scalar item arithmetic
    uint4 wa0 = make_uint4(0, 0, 0, 0), wb0 = wa0, wa1 = wa0, wb1 = wa0, wa2 = wa0, wb2 = wa0;
    Q8Pass q_cur = {}, q_nxt = {};
    bool q_chained = false;                      // the three fetches in flight are the first positions of the next pass
    bool q_nxt_valid = false;                    // there is a next pass (it may hold no item for this wavefront)
    int q_pos = 0, q_P = 3;                      // next position to fetch, positions of the current pass
    // This workgroup's slices: record `wg` first, then the records [sg_more, sg_more_end) named there.
    int sg_more = 0, sg_more_end = 0;
    auto q_make = [&](const uint32_t* bits, int rows, int words, int units, int row_end, int rb, int c0) -> Q8Pass {
        Q8Pass p;
        const int groups = (words + 15) >> 4;
        p.bits = bits;
        p.bytes = (uint32_t)((size_t)((rows + 31) >> 5) * groups * 2048);
        const int cu_n = min(min(units, chunk_cap), units - c0);
        p.ngroups = (cu_n + 3) >> 2;
        p.skip = groups - p.ngroups;
        const int nitems = p.ngroups * ((min(row_end - rb, kRowBlock) + 31) >> 5);
        const int per = mfma_items_per_wave(nitems, kWaves);
        p.it_begin = qwave * per;
        p.count = max(min(p.it_begin + per, nitems) - p.it_begin, 0);
        p.item_base = (rb >> 5) * groups + (c0 >> 2);
        return p;
    };
    // One fetch = position q_pos of [items of the current pass][idle positions up to q_P][first items of the next pass]:
    // always the same two load instructions, so that the compiler can count the fetches in flight.  Everything but
    // the lane's byte offset is wave-uniform (selected field by field and pinned to scalar registers).
    auto q_fetch_tiled = [&](uint4& wa, uint4& wb) {
        const bool in_cur = q_pos < q_P;
        const int j = in_cur ? q_pos : q_pos - q_P;
        const bool live = j < (in_cur ? q_cur.count : q_nxt.count);
        const int idx = (in_cur ? q_cur.it_begin : q_nxt.it_begin) + j;      // item of the pass: (row pair, unit group)
        const int ngroups = in_cur ? q_cur.ngroups : q_nxt.ngroups;
        const int skip = in_cur ? q_cur.skip : q_nxt.skip;                   // unit groups of the row outside the pass
        int item = (in_cur ? q_cur.item_base : q_nxt.item_base) + idx;
        if (skip != 0) item += (idx / ngroups) * skip;
        const uint64_t bits = (uint64_t)(in_cur ? q_cur.bits : q_nxt.bits);
        const uint32_t lo = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)bits);
        const uint32_t hi = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(bits >> 32));
        const uint32_t bytes = (uint32_t)__builtin_amdgcn_readfirstlane((int)(in_cur ? q_cur.bytes : q_nxt.bytes));
        const __amdgpu_buffer_rsrc_t rs = raw_buffer((const void*)(((uint64_t)hi << 32) | lo), bytes);
        const uint32_t soff = live ? (uint32_t)__builtin_amdgcn_readfirstlane(item) * 2048u : 0u;
        const uint32_t voff = live ? (uint32_t)qlane * 16u : kPastEnd;
        const u32x4_t a = __builtin_amdgcn_raw_buffer_load_b128(rs, voff, soff, 2 /* nt */);
        const u32x4_t b = __builtin_amdgcn_raw_buffer_load_b128(rs, voff + 1024u, soff, 2 /* nt */);
        wa = make_uint4(a.x, a.y, a.z, a.w);
        wb = make_uint4(b.x, b.y, b.z, b.w);
        ++q_pos;
    };

    {
        // SINGLE: one stage given by value, no tables and no counters; workgroup w takes rows
        // [w * single_rows, (w + 1) * single_rows)
#pragma unroll 1
        for (int sg = wg, nth = 0;; ++nth) {
            RunSegment seg;
            RunStage st;
            if constexpr (SINGLE) {
                seg = RunSegment{0, wg * single_rows, min(single.rows, (wg + 1) * single_rows), 0};
                st = single;
                if (nth || seg.row_end <= seg.row_begin) break;
            } else {
                if (nth) {
                    if (sg_more >= sg_more_end) break;
                    sg = sg_more++;
                }
                const RunSlice& sl = slices[sg];
                seg = sl.seg;
                st = sl.st;
                if (nth == 0) {
                    sg_more = sl.more_begin;
                    sg_more_end = sl.more_end;
                    if (seg.stage < 0) break;           // nothing for this workgroup
                }
                if (st.in_ext) st.in = ext_in;          // bound with the launch
                if (st.out_ext) st.out = ext_out;
            }
            const BitsView bv = bits_view(st);
            const int chunk_units = min(st.units, chunk_cap);
            const int upad = kQ8 ? q8_pitch(q8_units4(chunk_units)) : (chunk_units | 1);
            const bool one_chunk = chunk_units == st.units;
            float* xtot = xtot_base + kTotStride * (slice_count & 1);
            float* xtot_other = xtot_base + kTotStride * ((slice_count + 1) & 1);
            uint32_t* ebmax = ebmax_base + (slice_count & 1);
            ++slice_count;
            // kQ8: the unit scales (one dword per batch row and staged unit) sit in front of the pieces
            uint32_t* scl = (uint32_t*)xs_base;
            uint4* xs = xs_base + (kQ8 ? q8_scale_chunks(BATCH, q8_units4(chunk_units)) : 0);
            StageInput sin;
            sin.in = st.in; sin.s_col = st.s_col; sin.K = st.K; sin.in_stride = st.in_stride;
            sin.in_f32 = st.in_f32; sin.in_coherent = st.in_coherent; sin.vec_in = st.vec_in;

            // kQ8, row-major words: fetch cursor of this wavefront over its items = (pair of 16-row groups, 4-unit group)
            // of the current (row block, input chunk), unit group fastest
            int q_ngroups = 1, q_it_begin = 0, q_it_end = 0, q_it_f = 0, q_rp_f = 0, q_ub_f = 0, q_rb = 0, q_c0 = 0, q_cu_n = 0, q_nr = 0;
            auto q_setup = [&](int rb, int c0) {
                q_nr = min(seg.row_end - rb, kRowBlock);
                q_cu_n = min(chunk_units, st.units - c0);
                q_ngroups = (q_cu_n + 3) >> 2;
                const int nitems = q_ngroups * ((q_nr + 31) >> 5);
                const int per = mfma_items_per_wave(nitems, kWaves);
                q_it_begin = qwave * per;
                q_it_end = min(q_it_begin + per, nitems);
                q_it_f = q_it_begin;
                q_rp_f = q_it_begin / q_ngroups;
                q_ub_f = q_it_begin - q_rp_f * q_ngroups;
                q_rb = rb;
                q_c0 = c0;
            };
            auto q_fetch = [&](uint4& wa, uint4& wb) {
                const bool live = q_it_f < q_it_end;
                const int u = 4 * q_ub_f + (qlane >> 4);
                const int row = q_rb + 32 * q_rp_f + (qlane & 15);
                const bool ok = live && u < q_cu_n;
                wa = load_unit(bv, min(row, st.rows - 1), q_c0 + u, ok);
                wb = load_unit(bv, min(row + 16, st.rows - 1), q_c0 + u, ok);
                ++q_it_f;
                if (++q_ub_f == q_ngroups) { q_ub_f = 0; ++q_rp_f; }
            };
            // kQ8, tile order: the pass after (rb, c0) of this slice -- its next input chunk, its next row block, or the
            // first pass of this workgroup's next slice, whose description is fetched here, well ahead of its use
            RunSegment seg_n = seg;
            const uint32_t* bits_n = nullptr;
            int rows_n = 0, words_n = 0, units_n = 0;
            if constexpr (kQ8 && TILED && !SINGLE) {
                if (sg_more < sg_more_end) {
                    const RunSlice& sn = slices[sg_more];
                    seg_n = sn.seg;
                    bits_n = sn.st.bits; rows_n = sn.st.rows; words_n = sn.st.words; units_n = sn.st.units;
                }
            }
            auto q_has_next = [&](int rb, int c0) -> bool {
                return c0 + chunk_units < st.units || rb + kRowBlock < seg.row_end || bits_n != nullptr;
            };
            auto q_next_pass = [&](int rb, int c0) -> Q8Pass {
                if (c0 + chunk_units < st.units) return q_make(st.bits, st.rows, st.words, st.units, seg.row_end, rb, c0 + chunk_units);
                if (rb + kRowBlock < seg.row_end) return q_make(st.bits, st.rows, st.words, st.units, seg.row_end, rb + kRowBlock, 0);
                if (bits_n) return q_make(bits_n, rows_n, words_n, units_n, seg_n.row_end, seg_n.row_begin, 0);
                Q8Pass none = q_cur;             // no next pass: nothing of it is ever live
                none.count = 0;
                return none;
            };
            // Entering pass (rb, c0): its first three positions are already in flight (asked for by the previous pass)
            // or are asked for now.
            auto q_enter = [&](int rb, int c0) {
                q_cur = q_make(st.bits, st.rows, st.words, st.units, seg.row_end, rb, c0);
                q_P = (max(q_cur.count, 3) + 2) / 3 * 3;
                q_nxt = q_next_pass(rb, c0);
                q_pos = q_chained ? 3 : 0;
                q_nxt_valid = q_has_next(rb, c0);
                if (!q_chained) { q_fetch_tiled(wa0, wb0); q_fetch_tiled(wa1, wb1); q_fetch_tiled(wa2, wb2); }
            };
            if constexpr (kQ8) {
                // The packed words depend on nothing: the first three items of the slice are asked for before the
                // dependency wait and the staging of the input (in tile order: unless the previous pass already did),
                // and arrive while those run.
                if constexpr (OWN) {
                    // the first fetches are sent out after the staging
                } else if constexpr (TILED) {
                    if (!aborted) q_enter(seg.row_begin, 0);
                } else {
                    q_setup(seg.row_begin, 0);
                    q_fetch(wa0, wb0); q_fetch(wa1, wb1); q_fetch(wa2, wb2);
                }
            }

            if ((st.dep >= 0 || st.dep2 >= 0) && !aborted) {
                if (tid < kWave) {                               // wavefront 0 polls; lanes 0..7 own one sub-counter each
                    const unsigned long long gen = gen_raw / members;
                    unsigned spins = 0;
                    bool bad = false;
#pragma unroll 1
                    for (int which = 0; which < 2 && !bad; ++which) {
                        const int d = which ? st.dep2 : st.dep;
                        if (d < 0 || (which && st.addend_local)) continue;
                        const unsigned long long want = (gen + 1) * (unsigned long long)(which ? st.dep2_segs : st.dep_segs);
                        while (true) {
                            unsigned long long c = 0;
                            if (tid < kSubCounters)
                                c = __hip_atomic_load(counters + ((size_t)d * kSubCounters + tid) * kCounterStride,
                                                      __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                            c += __shfl_xor(c, 1, kWave);
                            c += __shfl_xor(c, 2, kWave);
                            c += __shfl_xor(c, 4, kWave);
                            const unsigned long long sum0 = __shfl(c, 0, kWave);
                            if (sum0 >= want) break;
                            __builtin_amdgcn_s_sleep(8);   // pollers must not crowd out the producers' atomics
                            unsigned flagged = 0;
                            if (tid == 0) flagged = __hip_atomic_load(status, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                            flagged = __shfl(flagged, 0, kWave);
                            if (++spins >= spin_limit || flagged) {
                                if (tid == 0) atomicOr(status, 1u);   // bounded wait: flag it, let the grid drain
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
            lds_barrier();                                       // s_flag; previous slice is done with xs / racc
            aborted = aborted || (s_flag != 0);
            // pairs 0 .. kWaves - 1 are the wavefronts' first ones; nobody takes a pair of the previous slice any more,
            // and the barrier behind the staging comes before the first one of this slice is taken
            if (OWN && tid == 0) s_pair = kWaves;
            if (tid < kTotStride) xtot_other[tid] = 0.f;         // every reader of it (the previous slice) is past the barrier
            if (DET && kQ8 && tid == 0) ebmax_base[slice_count & 1] = 0u;   // slice_count was advanced: this is the other one

            // rows row0 .. row0 + 3 of batch row b: row scale, bias, addend, store (as the epilogue of the row-block
            // loop).  The four rows of a lane are consecutive: 8-byte accesses where the alignment allows them.
            const bool vec_rows = (seg.row_begin & 3) == 0 && (st.out_stride & 3) == 0 &&
                                  ((((uintptr_t)st.s_row) | ((uintptr_t)st.bias) | ((uintptr_t)st.out)) & 7u) == 0;
            auto emit4 = [&](int row0, int b, float4_t v4) __attribute__((always_inline)) {
                float v[4] = {v4[0], v4[1], v4[2], v4[3]};   // scalars: a device-scope atomic store of a vector element stored element 0 four times
                const size_t o = (size_t)b * st.out_stride + row0;
                if (vec_rows && row0 + 3 < seg.row_end) {
                    if (st.s_row) {
                        const uint2 sw = *(const uint2*)(st.s_row + row0);
                        v[0] *= E::to_float((uint16_t)(sw.x & 0xFFFFu)); v[1] *= E::to_float((uint16_t)(sw.x >> 16));
                        v[2] *= E::to_float((uint16_t)(sw.y & 0xFFFFu)); v[3] *= E::to_float((uint16_t)(sw.y >> 16));
                    }
                    if (st.bias) {
                        const uint2 bw = *(const uint2*)(st.bias + row0);
                        v[0] += E::to_float((uint16_t)(bw.x & 0xFFFFu)); v[1] += E::to_float((uint16_t)(bw.x >> 16));
                        v[2] += E::to_float((uint16_t)(bw.y & 0xFFFFu)); v[3] += E::to_float((uint16_t)(bw.y >> 16));
                    }
                } else {
#pragma unroll
                    for (int k = 0; k < 4; ++k) {
                        if (row0 + k >= seg.row_end) break;
                        if (st.s_row) v[k] *= E::to_float(st.s_row[row0 + k]);
                        if (st.bias) v[k] += E::to_float(st.bias[row0 + k]);
                    }
                }
                if (st.addend) {
#pragma unroll
                    for (int k = 0; k < 4; ++k) {
                        if (row0 + k >= seg.row_end) break;
                        if (st.dep2 >= 0)
                            v[k] += __builtin_bit_cast(float, __hip_atomic_load((const uint32_t*)st.addend + o + k, __ATOMIC_RELAXED,
                                                                                __HIP_MEMORY_SCOPE_AGENT));
                        else
                            v[k] += st.addend[o + k];
                    }
                }
                if (!st.out_f32 && vec_rows && row0 + 3 < seg.row_end) {
                    uint2 pk;
                    pk.x = (uint32_t)E::from_float_clamped(v[0]) | ((uint32_t)E::from_float_clamped(v[1]) << 16);
                    pk.y = (uint32_t)E::from_float_clamped(v[2]) | ((uint32_t)E::from_float_clamped(v[3]) << 16);
                    *(uint2*)((uint16_t*)st.out + o) = pk;
                    return;
                }
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    if (row0 + k >= seg.row_end) break;
                    if (st.out_f32) {
                        // fp32 results (h, partial sums over terms) may be read by other workgroups of this launch:
                        // device-coherent store, completed before the counter of the slice is bumped
                        if (st.signal) __hip_atomic_store((uint32_t*)st.out + o + k, __builtin_bit_cast(uint32_t, v[k]),
                                                          __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                        else ((float*)st.out)[o + k] = v[k];
                    } else {
                        ((uint16_t*)st.out)[o + k] = E::from_float_clamped(v[k]);
                    }
                }
            };
            if constexpr (!kQ8) {
              if (!aborted) {
                // ---- 16-bit MFMA arithmetic (batch 8 and 16): wavefronts own whole row groups ----
                // A group = 16 consecutive rows of the slice (the rows of one MFMA).  In a round, wavefront w takes group
                // 16 * round + w and walks ALL columns of it, so a row sum lives in its MFMA accumulators from the first
                // column to the last and goes from there straight to the output: no row sums in LDS, no LDS atomics (at
                // batch 16 they cost more than the arithmetic), no barrier between rows, and results that do not depend
                // on any order left to the hardware.  With an input of one chunk the wavefronts of a workgroup meet once
                // per slice (after the staging) and the item fetches of a wavefront run on from group to group; with a
                // longer input the chunks are staged again for every round and the accumulators are kept across the
                // chunks of a round.  In the last round of a slice some wavefronts have no group.
                const int lane = tid & 63, r16 = lane & 15, g = lane >> 4;
                const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);       // scalar item arithmetic
                constexpr int kAccs = Pow2<DT>::kClasses;
                const int ngroups16 = (seg.row_end - seg.row_begin + 15) >> 4;
                const int rounds = (ngroups16 + kWaves - 1) / kWaves;            // the same for every wavefront
                // Few row groups (a short list gives a workgroup some tens of rows): the wavefronts that would have no
                // group take shares of the columns instead.  Wavefront w works on group w % groups, share w / groups of
                // every staged chunk; the shares of a group are added in share order by its first wavefront, through the
                // memory of the staged input once everybody is done with it.
                const bool split = rounds == 1 && 2 * ngroups16 <= kWaves;
                const int nshares = split ? kWaves / ngroups16 : 1;
                const int grp = split ? wave % ngroups16 : wave;                 // group of this wavefront in round 0
                const int share = split ? wave / ngroups16 : 0;                  // >= nshares: nothing to do
                const int my_rounds = split ? (share < nshares ? 1 : 0)
                                            : (ngroups16 > wave ? (ngroups16 - wave + kWaves - 1) / kWaves : 0);
                float4_t acc[kAccs];
#pragma unroll
                for (int k = 0; k < kAccs; ++k) acc[k] = (float4_t){0.f, 0.f, 0.f, 0.f};
                // the q-th group of this wavefront is complete: acc[v] = sum for its row 4 g + v, batch row r16
                auto store_group = [&](int q, const float4_t& bsum) __attribute__((always_inline)) {
                    const float4_t sum = bsum * -2.f;                             // signed sum = (sum of x) - 2 (sum of b x)
                    if (r16 < BATCH) {
                        const float xt = xtot[r16];
                        const int row0 = seg.row_begin + 16 * (grp + kWaves * q) + 4 * g;
                        if (row0 < seg.row_end) emit4(row0, r16, sum + xt);
                    }
                };
                // The same for a whole group whose results need nothing but their row scale (no bias, no addend, 8-byte
                // aligned rows), without a load or a varying number of stores among the lane memory operations, so that
                // the item fetches in flight need not be waited for: the 16 scales come through the scalar cache, the
                // results leave as two buffer stores per lane, one per output type, past the end of the buffer for the
                // other type and for the lanes that hold no batch row.
                const int nrows16 = seg.row_end - seg.row_begin;
                const size_t out_elems = (size_t)(BATCH - 1) * st.out_stride + st.rows;
                const bool plain_out = vec_rows && st.s_row && !st.bias && !st.addend && out_elems < (1u << 28);
                const __amdgpu_buffer_rsrc_t rout = raw_buffer(st.out, (uint32_t)(out_elems * (st.out_f32 ? 4u : 2u)));
                const uint32_t past32 = st.out_f32 ? 0u : kPastEnd, past16 = st.out_f32 ? kPastEnd : 0u;
                auto store_group_plain = [&](int grow, const float4_t& bsum) __attribute__((always_inline)) {
                    typedef const uint32_t __attribute__((address_space(4)))* scalar_words_t;
                    const int prow = seg.row_begin + __builtin_amdgcn_readfirstlane(grow);
                    const scalar_words_t sp = (scalar_words_t)(uintptr_t)(st.s_row + prow);
                    uint32_t sw[8];
#pragma unroll
                    for (int i = 0; i < 8; ++i) {
                        sw[i] = sp[i];
                        asm volatile("" : "+s"(sw[i]));                  // kept in scalar registers: one scalar load each
                    }
                    uint32_t s0 = sw[0], s1 = sw[1];                     // rows 4g .. 4g + 3
#pragma unroll
                    for (int q = 1; q < 4; ++q) {
                        s0 = g == q ? sw[2 * q] : s0;
                        s1 = g == q ? sw[2 * q + 1] : s1;
                    }
                    float4_t v = bsum * -2.f + xtot[min(r16, BATCH - 1)];
                    v[0] *= E::to_float((uint16_t)(s0 & 0xFFFFu)); v[1] *= E::to_float((uint16_t)(s0 >> 16));
                    v[2] *= E::to_float((uint16_t)(s1 & 0xFFFFu)); v[3] *= E::to_float((uint16_t)(s1 >> 16));
                    const bool live = r16 < BATCH;
                    const uint32_t elem = (uint32_t)min(r16, BATCH - 1) * (uint32_t)st.out_stride + (uint32_t)(prow + 4 * g);
                    const uint32_t o32 = live ? (elem * 4u) | past32 : kPastEnd;
                    const uint32_t o16 = live ? (elem * 2u) | past16 : kPastEnd;
                    const u32x4_t f = {as_bits(v[0]), as_bits(v[1]), as_bits(v[2]), as_bits(v[3])};
                    __builtin_amdgcn_raw_buffer_store_b128(f, rout, o32, 0, kCacheAgentCoherent);   // fp32: read by other workgroups
                    const u32x2_t h = {(uint32_t)E::from_float_clamped(v[0]) | ((uint32_t)E::from_float_clamped(v[1]) << 16),
                                       (uint32_t)E::from_float_clamped(v[2]) | ((uint32_t)E::from_float_clamped(v[3]) << 16)};
                    __builtin_amdgcn_raw_buffer_store_b64(h, rout, o16, 0, kCacheDefault);
                };
                // The groups [q_begin, q_end) of this wavefront times the unit groups of the staged chunk (c0, cu_n).
                // Items = (row group, 4-unit group), unit group fastest.  Three item fetches (1 KB of packed words each) in
                // flight, in three register sets that take turns, each refilled right after its use; a row group is
                // walked in a multiple of three positions (the last ones may be empty), so the register sets keep their
                // turns from group to group and the fetches run on into the next group while the current one is finished
                // and stored.  A fetch past the last item loads nothing (offset past the end).  `complete`: the staged
                // chunk is the last of the input.
                auto run_items = [&](auto order_c, int q_begin, int q_end, int c0, int cu_n, bool complete) __attribute__((always_inline)) {
                    constexpr int kOrder = decltype(order_c)::value;      // one copy of the loop per word order: see load_unit
                    const int ngroups_all = (cu_n + 3) >> 2;
                    const int j_begin = split ? share * ngroups_all / nshares : 0;        // this wavefront's unit groups
                    const int ngroups = (split ? (share + 1) * ngroups_all / nshares : ngroups_all) - j_begin;
                    const int positions = (ngroups + 2) / 3 * 3;
                    // the last round has groups for some wavefronts only, and a chunk may have fewer unit groups than shares
                    const int nq = ngroups > 0 ? max(min(q_end, my_rounds) - q_begin, 0) : 0;
                    int f_left = nq * positions, f_q = q_begin, f_j = 0;  // fetch cursor
                    auto fetch = [&](uint4& w) {
                        if constexpr (kOrder == 1) {
                            // tile order: the item is one half (1 KB) of a 2 KB tile (slices begin at multiples of 16
                            // rows, chunks at multiples of 4 units), 16 bytes per lane; rows and units past the end are
                            // zero words
                            const bool ok = f_left > 0 && f_j < ngroups;
                            const int half = (seg.row_begin >> 4) + grp + kWaves * f_q;
                            const int off = ((half >> 1) * bv.groups + (c0 >> 2) + j_begin + f_j) * 2048 + (half & 1) * 1024;
                            const uint32_t soff = ok ? (uint32_t)__builtin_amdgcn_readfirstlane(off) : 0u;
                            const uint32_t voff = ok ? (uint32_t)lane * 16u : kPastEnd;
                            const u32x4_t a = __builtin_amdgcn_raw_buffer_load_b128(bv.rsrc, voff, soff, 2 /* nt */);
                            w = make_uint4(a.x, a.y, a.z, a.w);
                        } else {
                            const int u = 4 * (j_begin + f_j) + g;
                            const int row = seg.row_begin + 16 * (grp + kWaves * f_q) + r16;
                            w = load_unit<kOrder>(bv, min(row, st.rows - 1), c0 + u, f_left > 0 && u < cu_n);   // u < cu_n fails on empty positions as well
                        }
                        --f_left;
                        if (++f_j == positions) { f_j = 0; ++f_q; }
                    };
                    auto work = [&](uint4& w, int j) {
                        const int u = 4 * (j_begin + j) + g;
                        if constexpr (kOrder == 2) trim_unit(bv, w, c0 + u);   // tile order pads with zero words
                        unit_mfma_pow2<DT, BATCH>(w, xs, upad, min(u, cu_n - 1), acc);   // w = 0 beyond cu_n
                    };
                    // A full wait ahead of the first fetches (what the staging loaded has been used) and after the stores
                    // of a group: inside the loop the item fetches are the only accesses in flight and the compiler waits
                    // for the oldest of them only, not for all.
                    __builtin_amdgcn_s_waitcnt(0);
                    uint4 w0, w1, w2;
                    fetch(w0);
                    fetch(w1);
                    fetch(w2);
#pragma unroll 1
                    for (int q = q_begin; q < q_begin + nq; ++q) {
#pragma unroll 1
                        for (int j = 0; j < positions; j += 3) {
                            work(w0, j);
                            fetch(w0);
                            if (j + 1 < ngroups) work(w1, j + 1);
                            fetch(w1);
                            if (j + 2 < ngroups) work(w2, j + 2);
                            fetch(w2);
                        }
                        if (complete && !split) {
                            const int grow = 16 * (grp + kWaves * q);
                            if (plain_out && grow + 16 <= nrows16) {
                                store_group_plain(grow, pow2_combine<DT>(acc));
                            } else {
                                store_group(q, pow2_combine<DT>(acc));
                                __builtin_amdgcn_s_waitcnt(0);           // loads and a varying number of stores behind the fetches
                            }
#pragma unroll
                            for (int k = 0; k < kAccs; ++k) acc[k] = (float4_t){0.f, 0.f, 0.f, 0.f};
                        }
                    }
                };
                bool staged = false;                                      // a chunk is staged and may be in use
                float* unit_tot = racc;                                   // [BATCH][upad] totals of the staged units
                auto stage_chunk = [&](int c0, int cu_n) __attribute__((always_inline)) {
                    if (staged) {
                        lds_barrier();                                    // every wavefront is done with the staged chunk and the totals
                        if (c0 == 0) {
                            if (tid < kTotStride) xtot[tid] = 0.f;        // staged again from the first column: the totals start over
                            lds_barrier();
                        }
                    }
                    // unit totals to LDS, then 16 lanes per batch row add them in a fixed order
                    stage_units_rows<DT, BATCH, kStreamThreads>(xs, unit_tot, sin, c0, cu_n, upad);
                    lds_barrier();
                    if (tid < BATCH * 16) {                               // whole wavefronts
                        const int b = tid >> 4, k = tid & 15;
                        float t = 0.f;
                        for (int cu = k; cu < cu_n; cu += 16) t += unit_tot[b * upad + cu];
                        t = group_sum(t, 16);
                        if (k == 0) xtot[b] += t;
                    }
                    staged = true;
                    lds_barrier();                                        // staged input and its totals visible
                };
                auto owned = [&](int q_begin, int q_end, int c0, int cu_n, bool complete) __attribute__((always_inline)) {
                    if (bv.groups) run_items(std::integral_constant<int, 1>{}, q_begin, q_end, c0, cu_n, complete);
                    else run_items(std::integral_constant<int, 2>{}, q_begin, q_end, c0, cu_n, complete);
                    if (split && complete) {
                        float4_t mine = pow2_combine<DT>(acc);
                        float4_t* shares = (float4_t*)xs;                 // (kWaves - 1) x 64 x 16 bytes
                        lds_barrier();                                    // every wavefront is done with the staged input
                        if (share > 0 && share < nshares) shares[(wave - ngroups16) * 64 + lane] = mine;
                        lds_barrier();
                        if (share == 0) {
                            for (int t = 1; t < nshares; ++t) mine += shares[(grp + (t - 1) * ngroups16) * 64 + lane];
                            store_group(0, mine);
                        }
                    }
                };
                // an input of one chunk is staged once and every wavefront walks all its groups in one go
                const int staged_rounds = one_chunk ? min(rounds, 1) : rounds;
#pragma unroll 1
                for (int r = 0; r < staged_rounds; ++r) {
#pragma unroll 1
                    for (int c0 = 0; c0 < st.units; c0 += chunk_units) {
                        const int cu_n = min(chunk_units, st.units - c0);
                        stage_chunk(c0, cu_n);
                        owned(one_chunk ? 0 : r, one_chunk ? rounds : r + 1, c0, cu_n, c0 + chunk_units >= st.units);
                    }
                }
              }
            } else if (OWN && !aborted) {
                // ---- fp4 x fp8 arithmetic, wavefronts own row pairs (every input is one chunk) ----
                if constexpr (OWN) {
                    const int cu_n = st.units;
                    // DET: the input totals are kept per wavefront and added in wavefront order below; the row sums are
                    // formed by one wavefront in a fixed order whichever wavefront takes the pair, so nothing is rounded
                    // to a grid here
                    stage_units_q8<DT, BATCH, THREADS, DET>(xs, scl, xtot, sin, 0, cu_n, upad, ebmax);
                    lds_barrier();                               // staged input and its totals visible
                    const int r16 = qlane & 15, g = qlane >> 4;
                    const int nrows = seg.row_end - seg.row_begin;
                    const int npairs = (nrows + 31) >> 5;
                    const int ngroups = (cu_n + 3) >> 2;
                    constexpr int kOwnDepth = 3;                       // item fetches in flight per wavefront
                    const int positions = (ngroups + kOwnDepth - 1) / kOwnDepth * kOwnDepth;   // the register pairs keep their turns from pair to pair
                    // results that need only their row scale go out as buffer stores (see the end of a pair)
                    const size_t out_elems = (size_t)(BATCH - 1) * st.out_stride + st.rows;
                    const bool plain_out = vec_rows && (nrows & 31) == 0 && st.s_row && !st.bias && !st.addend && out_elems < (1u << 28);
                    const __amdgpu_buffer_rsrc_t rout = raw_buffer(st.out, (uint32_t)(out_elems * (st.out_f32 ? 4u : 2u)));
                    const int groups_all = (st.words + 15) >> 4;      // tiles per row pair in memory
                    const uint32_t bits_bytes = (uint32_t)((size_t)((st.rows + 31) >> 5) * groups_all * 2048);
                    const __amdgpu_buffer_rsrc_t rs = raw_buffer(st.bits, bits_bytes);
                    const int tile0 = (seg.row_begin >> 5) * groups_all;
                    // operand column of this lane (batch row, piece), as in the row-block loop below
                    const bool qlive = r16 < BATCH * kQ8Pieces;
                    const int qcol = min(r16, BATCH * kQ8Pieces - 1);
                    const uint4* qbase = xs + (size_t)qcol * upad + 8 * (g >> 1) + (g & 1);
                    const uint32_t* qscl = scl + (qcol / kQ8Pieces) * ((upad - 1) >> 3) + g;
                    const bool qlast = qlive && r16 % kQ8Pieces == kQ8Pieces - 1;
                    // Pairs: the one being worked on, and up to two that the fetches have already moved on to.
                    int c_pair = qwave, f_pair = qwave, f_j = 0;
                    int next_a = 0, next_b = 0, queued = 0;
                    auto take_pair = [&]() -> int {
                        int p = 0;
                        if (qlane == 0) p = atomicAdd(&s_pair, 1);
                        return __builtin_amdgcn_readfirstlane(p);
                    };
                    auto fetch = [&](uint4& wa, uint4& wb) __attribute__((always_inline)) {
                        const bool live = f_pair < npairs && f_j < ngroups;
                        const int tile = tile0 + f_pair * groups_all + f_j;
                        const uint32_t soff = live ? (uint32_t)__builtin_amdgcn_readfirstlane(tile) * 2048u : 0u;
                        const uint32_t voff = live ? (uint32_t)qlane * 16u : kPastEnd;
                        const u32x4_t a = __builtin_amdgcn_raw_buffer_load_b128(rs, voff, soff, 2 /* nt */);
                        const u32x4_t b = __builtin_amdgcn_raw_buffer_load_b128(rs, voff + 1024u, soff, 2 /* nt */);
                        wa = make_uint4(a.x, a.y, a.z, a.w);
                        wb = make_uint4(b.x, b.y, b.z, b.w);
                        if (++f_j == positions) {
                            f_j = 0;
                            f_pair = f_pair < npairs ? take_pair() : npairs;
                            if (queued == 0) next_a = f_pair; else next_b = f_pair;
                            ++queued;
                        }
                    };
                    Q8Operand opnd = {};
                    int qscale = 0x7F7F7F7F;
                    float4_t acc_a = {0.f, 0.f, 0.f, 0.f}, acc_b = {0.f, 0.f, 0.f, 0.f};
                    auto work = [&](uint4& wa, uint4& wb, int ub) __attribute__((always_inline)) {
                        if (qlive) {
                            q8_read_operand(opnd, qbase + 32 * ub);
                            qscale = (int)qscl[4 * ub];
                        }
                        unit_mfma_q8_pair(wa, wb, opnd, qscale, acc_a, acc_b);
                    };
                    auto three_items = [&](int j) __attribute__((always_inline)) {
                        work(wa0, wb0, j);
                        fetch(wa0, wb0);
                        if (j + 1 < ngroups) work(wa1, wb1, j + 1);
                        fetch(wa1, wb1);
                        if constexpr (kOwnDepth == 3) {
                            if (j + 2 < ngroups) work(wa2, wb2, j + 2);
                            fetch(wa2, wb2);
                        }
                    };
                    // PLAIN: every pair of the slice is whole and nothing but the row scale is applied on the way out.
                    // The scales then come through the scalar cache (64 bytes per pair, the same for every lane) and the
                    // results leave as four buffer stores per lane (two per output type, past the end of the buffer for
                    // the other type and for the lanes that hold no sum): no load among the lane memory operations of
                    // the loop but the item fetches, and a fixed number of stores on every way through it, so the
                    // compiler, which counts the lane memory operations behind a fetch to know how long to wait for it,
                    // lets the fetches in flight stay in flight from pair to pair.  (A load at the end of a pair waits
                    // for all of them, and so does every step of the loop behind a varying number of stores.)  For the
                    // same reason the first three items of a pair are code of their own, reached only with four stores
                    // behind the three fetches: from the end of a pair and from the start of the slice.
                    // (That holds at batch 4.  At one and two batch rows the same loop without the code of its own, where
                    // the first items of a pair wait for a fetch more than they need, measures 5 % faster and equal.)
                    constexpr bool kOwnExactWaits = BATCH >= 4;
                    auto run_pairs = [&](auto plain_tag) __attribute__((always_inline)) {
                        constexpr bool PLAIN = decltype(plain_tag)::value;
                        const uint32_t past32 = st.out_f32 ? 0u : kPastEnd, past16 = st.out_f32 ? kPastEnd : 0u;
                        auto store_pair = [&](uint32_t elem, bool live, float4_t va, float4_t vb) __attribute__((always_inline)) {
                            const uint32_t o32 = live ? (elem * 4u) | past32 : kPastEnd;
                            const uint32_t o16 = live ? (elem * 2u) | past16 : kPastEnd;
                            // fp32 results may be read by other workgroups of this launch: device-coherent stores
                            const u32x4_t fa = {as_bits(va[0]), as_bits(va[1]), as_bits(va[2]), as_bits(va[3])};
                            const u32x4_t fb = {as_bits(vb[0]), as_bits(vb[1]), as_bits(vb[2]), as_bits(vb[3])};
                            __builtin_amdgcn_raw_buffer_store_b128(fa, rout, o32, 0, kCacheAgentCoherent);
                            __builtin_amdgcn_raw_buffer_store_b128(fb, rout, o32 + 64u, 0, kCacheAgentCoherent);
                            const u32x2_t ha = {(uint32_t)E::from_float_clamped(va[0]) | ((uint32_t)E::from_float_clamped(va[1]) << 16),
                                                (uint32_t)E::from_float_clamped(va[2]) | ((uint32_t)E::from_float_clamped(va[3]) << 16)};
                            const u32x2_t hb = {(uint32_t)E::from_float_clamped(vb[0]) | ((uint32_t)E::from_float_clamped(vb[1]) << 16),
                                                (uint32_t)E::from_float_clamped(vb[2]) | ((uint32_t)E::from_float_clamped(vb[3]) << 16)};
                            __builtin_amdgcn_raw_buffer_store_b64(ha, rout, o16, 0, kCacheDefault);
                            __builtin_amdgcn_raw_buffer_store_b64(hb, rout, o16 + 32u, 0, kCacheDefault);
                        };
                        __builtin_amdgcn_s_waitcnt(0);           // what the staging loaded has been used: see the tile-order loop below
                        fetch(wa0, wb0); fetch(wa1, wb1);
                        if constexpr (kOwnDepth == 3) fetch(wa2, wb2);
                        if constexpr (PLAIN) store_pair(0u, false, acc_a, acc_b);
#pragma unroll 1
                        while (c_pair < npairs) {
                            if constexpr (PLAIN && kOwnExactWaits) three_items(0);
#pragma unroll 1
                            for (int j = PLAIN && kOwnExactWaits ? kOwnDepth : 0; j < positions; j += kOwnDepth) three_items(j);
                            // acc_a[v]: row 32 pair + 4 g + v (acc_b: 16 rows further), column r16; the sum over the pieces
                            // of a batch row is valid in the lane of its last piece
                            float4_t sa, sb;
#pragma unroll
                            for (int v = 0; v < 4; ++v) {
                                sa[v] = q8_piece_sum(acc_a[v]);
                                sb[v] = q8_piece_sum(acc_b[v]);
                            }
                            const int b = qcol / kQ8Pieces;
                            float xt = 0.f;
                            if constexpr (DET) {
#pragma unroll
                                for (int w = 0; w < kWaves; ++w) xt += xtot[4 * w + b];
                            } else {
                                xt = xtot[b];
                            }
                            sa += xt;
                            sb += xt;
                            if constexpr (PLAIN) {
                                typedef const uint32_t __attribute__((address_space(4)))* scalar_words_t;
                                const int prow = seg.row_begin + 32 * __builtin_amdgcn_readfirstlane(c_pair);
                                const scalar_words_t sp = (scalar_words_t)(uintptr_t)(st.s_row + prow);
                                uint32_t sw[16];
#pragma unroll
                                for (int i = 0; i < 16; ++i) {
                                    sw[i] = sp[i];
                                    asm volatile("" : "+s"(sw[i]));      // kept in scalar registers: one scalar load each
                                }
                                uint32_t s0 = sw[0], s1 = sw[1], s2 = sw[8], s3 = sw[9];   // rows 4g .. 4g + 3, 16 + 4g .. 16 + 4g + 3
#pragma unroll
                                for (int q = 1; q < 4; ++q) {
                                    s0 = g == q ? sw[2 * q] : s0;
                                    s1 = g == q ? sw[2 * q + 1] : s1;
                                    s2 = g == q ? sw[8 + 2 * q] : s2;
                                    s3 = g == q ? sw[9 + 2 * q] : s3;
                                }
                                sa[0] *= E::to_float((uint16_t)(s0 & 0xFFFFu)); sa[1] *= E::to_float((uint16_t)(s0 >> 16));
                                sa[2] *= E::to_float((uint16_t)(s1 & 0xFFFFu)); sa[3] *= E::to_float((uint16_t)(s1 >> 16));
                                sb[0] *= E::to_float((uint16_t)(s2 & 0xFFFFu)); sb[1] *= E::to_float((uint16_t)(s2 >> 16));
                                sb[2] *= E::to_float((uint16_t)(s3 & 0xFFFFu)); sb[3] *= E::to_float((uint16_t)(s3 >> 16));
                                store_pair((uint32_t)b * (uint32_t)st.out_stride + (uint32_t)(prow + 4 * g), qlast, sa, sb);
                            } else {
                                if (qlast) {
                                    const int row0 = seg.row_begin + 32 * c_pair + 4 * g;
                                    if (row0 < seg.row_end) emit4(row0, b, sa);
                                    if (row0 + 16 < seg.row_end) emit4(row0 + 16, b, sb);
                                }
                                __builtin_amdgcn_s_waitcnt(0);   // loads and a varying number of stores: start over with only fetches in flight
                            }
                            acc_a = acc_b = (float4_t){0.f, 0.f, 0.f, 0.f};
                            c_pair = next_a;
                            next_a = next_b;
                            --queued;
                        }
                    };
                    if (plain_out) run_pairs(std::true_type{});
                    else run_pairs(std::false_type{});
                }
            } else if (!aborted) {
                bool staged = false;
#pragma unroll 1
                for (int rb = seg.row_begin; rb < seg.row_end; rb += kRowBlock) {
                    const int nr = min(seg.row_end - rb, kRowBlock);
                    for (int i = tid; i < nr * BATCH; i += kStreamThreads) {
                        racc[i] = 0.f;
                        if constexpr (DET) rtot[i] = 0.f;
                    }
#pragma unroll 1
                    for (int c0 = 0; c0 < st.units; c0 += chunk_units) {
                        const int cu_n = min(chunk_units, st.units - c0);
                        if (!(one_chunk && staged)) {
                            if (c0) lds_barrier();
                            if (kTotals && c0 == 0 && staged) {
                                // the input is staged again for a further row block: the totals start over (the first
                                // staging of a slice finds them cleared a barrier ahead); every reader of the previous
                                // totals has passed a barrier by now
                                if (tid < kTotStride) xtot[tid] = 0.f;
                                if (DET && tid == 0) *ebmax = 0u;
                                lds_barrier();
                            }
                            if constexpr (kQ8) stage_units_q8<DT, BATCH, THREADS, DET>(xs, scl, xtot, sin, c0, cu_n, upad, ebmax);
                            staged = true;
                        }
                        lds_barrier();                           // xs / xsum / zeroed racc visible
                        if constexpr (kQ8) {
                            // Items = (pair of 16-row groups, 4-unit group), unit group fastest: one read of the input
                            // operand (eight 16-byte LDS reads per lane) serves two row groups, and a wavefront takes a
                            // contiguous run of items, so it adds its two accumulators to the row sums only when the
                            // pair changes (LDS float atomics cost about 2.5 cycles per lane).
                            const int r16 = qlane & 15, g = qlane >> 4;
                            if (rb != seg.row_begin || c0 != 0) {        // the first pass was set up ahead of the wait
                                if constexpr (TILED) {
                                    q_enter(rb, c0);
                                } else {
                                    q_setup(rb, c0);
                                    q_fetch(wa0, wb0); q_fetch(wa1, wb1); q_fetch(wa2, wb2);
                                }
                            }
                            const int ngroups = TILED ? q_cur.ngroups : q_ngroups;
                            const int it_begin = TILED ? q_cur.it_begin : q_it_begin;
                            const int it_end = TILED ? q_cur.it_begin + q_cur.count : q_it_end;
                            // operand column of this lane (batch row, piece) and its first chunk; columns beyond the
                            // last piece are never read back, so their lanes skip the LDS reads (40 % less LDS time)
                            const bool qlive = r16 < BATCH * kQ8Pieces;
                            const int qcol = min(r16, BATCH * kQ8Pieces - 1);
                            const uint4* qbase = xs + (size_t)qcol * upad + 8 * (g >> 1) + (g & 1);
                            // the lane's block scale: the four class bytes of unit 4 ub + g of its batch row
                            const uint32_t* qscl = scl + (qcol / kQ8Pieces) * ((upad - 1) >> 3) + g;
                            const bool qlast = qlive && r16 % kQ8Pieces == kQ8Pieces - 1;   // holds the sum over the pieces
                            float* rdst = racc + (4 * g) * BATCH + qcol / kQ8Pieces;
                            int rp = it_begin / ngroups, ub = it_begin - rp * ngroups;      // compute cursor
                            Q8Operand opnd = {};
                            int qscale = 0x7F7F7F7F;
                            float4_t acc_a = {0.f, 0.f, 0.f, 0.f}, acc_b = {0.f, 0.f, 0.f, 0.f};
                            int rp_run = rp;
                            // DET: 1.5 * 2^k with 2^(k-1) above every partial and complete row sum of this chunk:
                            // (columns) x (largest staged value) x 2 (classes 0..2 count twice, the totals make up for it)
                            float det_c = 0.f;
                            if constexpr (DET) {
                                const uint32_t cols = (uint32_t)q8_units4(cu_n) * 128u;
                                const uint32_t e = min(*ebmax + (32u - (uint32_t)__builtin_clz(cols - 1u)) + 3u, 254u);
                                det_c = as_float((e << 23) | 0x400000u);
                            }
                            auto flush = [&]() {
                                // acc[v] = partial sum of row 32 rp_run + 4 g + v (acc_b: 16 rows further) for column r16
#pragma unroll
                                for (int v = 0; v < 4; ++v) {
                                    float sa = q8_piece_sum(acc_a[v]), sb = q8_piece_sum(acc_b[v]);
                                    if constexpr (DET) {
                                        sa = grid_round(sa, det_c);
                                        sb = grid_round(sb, det_c);
                                    }
                                    const int row = 32 * rp_run + 4 * g + v;
                                    if (qlast && row < nr) atomicAdd(&rdst[(32 * rp_run + v) * BATCH], sa);
                                    if (qlast && row + 16 < nr) atomicAdd(&rdst[(32 * rp_run + 16 + v) * BATCH], sb);
                                }
                            };
                            auto work = [&](uint4& wa, uint4& wb) {
                                if (rp != rp_run) {
                                    flush();
                                    acc_a = acc_b = (float4_t){0.f, 0.f, 0.f, 0.f};
                                    rp_run = rp;
                                }
                                if (qlive) {
                                    q8_read_operand(opnd, qbase + 32 * ub);
                                    qscale = (int)qscl[4 * ub];
                                }
                                if constexpr (!TILED) {
                                    trim_unit(bv, wa, c0 + 4 * ub + g);   // w = 0 beyond cu_n, padding staged as 0
                                    trim_unit(bv, wb, c0 + 4 * ub + g);
                                }
                                unit_mfma_q8_pair(wa, wb, opnd, qscale, acc_a, acc_b);
                                if (++ub == ngroups) { ub = 0; ++rp; }
                            };
                            // three register pairs in rotation, each refilled right after its use: nothing in flight
                            // is ever copied
                            static_assert(kQ8Depth == 3, "the rotation below is written out for three register pairs");
                            if constexpr (TILED) {
                                const int count = q_cur.count;
                                // A full wait ahead of the loop (what is in flight was asked for a staging ago and has
                                // arrived): without it the compiler carries the possibility of an outstanding generic-
                                // address access (staging fallback, epilogue) into the loop and waits for ALL fetches at
                                // every step instead of for the oldest one.
                                __builtin_amdgcn_s_waitcnt(0);
#pragma unroll 1
                                for (int i = 0; i < q_P; i += kQ8Depth) {
                                    if (i < count) work(wa0, wb0);
                                    q_fetch_tiled(wa0, wb0);
                                    if (i + 1 < count) work(wa1, wb1);
                                    q_fetch_tiled(wa1, wb1);
                                    if (i + 2 < count) work(wa2, wb2);
                                    q_fetch_tiled(wa2, wb2);
                                }
                                q_chained = q_nxt_valid;                 // what is in flight now belongs to the next pass
                            } else {
                                auto step = [&](uint4& wa, uint4& wb) {
                                    work(wa, wb);
                                    q_fetch(wa, wb);
                                };
                                int it = it_begin;
#pragma unroll 1
                                for (; it + kQ8Depth <= it_end; it += kQ8Depth) {
                                    step(wa0, wb0); step(wa1, wb1); step(wa2, wb2);
                                }
                                if (it < it_end) step(wa0, wb0);
                                if (it + 1 < it_end) step(wa1, wb1);
                            }
                            if (it_begin < it_end) flush();              // + the staged total of classes 0..2 at the end
                            if constexpr (DET) {
                                if (!one_chunk) {
                                    // the next input chunk has a grid of its own: its sums are added to what the chunks
                                    // so far came to, element by element (the loop top or the barrier below orders this
                                    // against the next partial sums)
                                    lds_barrier();
                                    for (int i = tid; i < nr * BATCH; i += kStreamThreads) {
                                        rtot[i] += racc[i];
                                        racc[i] = 0.f;
                                    }
                                }
                            }
                        }
                        }
                    lds_barrier();                               // row sums complete
                    for (int i = tid; i < nr * BATCH; i += kStreamThreads) {
                        const int row = rb + i / BATCH, b = i % BATCH;
                        float v = racc[i];
                        if constexpr (DET) {
                            if (!one_chunk) v += rtot[i];
                            float xt = 0.f;
#pragma unroll
                            for (int w = 0; w < kWaves; ++w) xt += xtot[4 * w + b];   // wavefront order
                            v += xt;
                        } else if constexpr (kTotals) {
                            v += xtot[b];
                        }
                        if (st.s_row) v *= E::to_float(st.s_row[row]);
                        if (st.bias) v += E::to_float(st.bias[row]);
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
                            if (st.signal) __hip_atomic_store((uint32_t*)st.out + o, __builtin_bit_cast(uint32_t, v),
                                                              __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                            else ((float*)st.out)[o] = v;
                        } else {
                            ((uint16_t*)st.out)[o] = E::from_float_clamped(v);
                        }
                    }
                    if (rb + kRowBlock < seg.row_end) lds_barrier();   // racc is zeroed again next
                }
            }

            if (st.signal) {
                // Every wavefront waits until its own stores above have been acknowledged by the memory side (a
                // workgroup-scope fence emits no such wait on this target, and nothing orders the stores of one
                // wavefront against the counter add of another), then the barrier collects all of them.
                asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
                __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
                __syncthreads();
                if (tid == 0) {
                    unsigned long long* c =
                        counters + ((size_t)seg.stage * kSubCounters + (wg & (kSubCounters - 1))) * kCounterStride;
                    if (st.heavy_release) __hip_atomic_fetch_add(c, 1ull, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_AGENT);
                    else __hip_atomic_fetch_add(c, 1ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                }
            }
        }
    }

    if (tid == 0 && !SINGLE) {
        unsigned long long* exit_sub = counters + (size_t)nstages * kSubCounters * kCounterStride;
        __hip_atomic_fetch_add(exit_sub + (size_t)(wg & (kExitSubs - 1)) * kCounterStride, 1ull, __ATOMIC_RELAXED,
                               __HIP_MEMORY_SCOPE_AGENT);
    }
}

size_t stream_counter_bytes(int nstages) {
    return ((size_t)nstages * kSubCounters + kExitSubs) * kCounterStride * sizeof(unsigned long long);
}

// ---- host side --------------------------------------------------------------------------------
static void stream_lds_plan(int batch, int arith, int max_units, int* chunk_cap_out, size_t* lds_out, bool det = false,
                            bool own = false) {
    const int racc_bytes = (int)stream_head_bytes(batch, arith, det && arith == 2, own && arith == 2);
    if (arith == 2) {
        // kQ8Pieces bytes per column and batch row, staged in whole groups of four units
        // plus one scale dword per batch row and unit
        int chunk_cap = (kStreamLdsMax - racc_bytes - batch * kQ8Pieces * (int)sizeof(uint4) - 16) / (batch * (kQ8Pieces * 128 + 4));
        chunk_cap &= ~3;
        const int chunk_units = max_units < chunk_cap ? max_units : chunk_cap;
        *chunk_cap_out = chunk_cap;
        *lds_out = (size_t)racc_bytes + (size_t)(q8_scale_chunks(batch, q8_units4(chunk_units)) + q8_chunks(batch, q8_units4(chunk_units))) * sizeof(uint4);
        return;
    }
    int chunk_cap = (kStreamLdsMax - racc_bytes - batch * (int)sizeof(uint4)) / (batch * 16 * (int)sizeof(uint4));
    chunk_cap = (chunk_cap - 1) & ~3;   // whole 4-unit groups, and room for the odd pitch chunk_units | 1
    const int chunk_units = max_units < chunk_cap ? max_units : chunk_cap;
    *chunk_cap_out = chunk_cap;
    // the staged input's memory also takes the column shares of a slice of few rows: 1 KB per wavefront but the first
    size_t xs_bytes = (size_t)xs_chunks(batch, chunk_units | 1) * sizeof(uint4);
    if (xs_bytes < kStreamShareBytes) xs_bytes = kStreamShareBytes;
    *lds_out = (size_t)racc_bytes + xs_bytes;
}

// Which arithmetic, by batch.  The fp4 x fp8 arithmetic (ARITH 2) is three times cheaper per packed bit than the
// 16-bit MFMA operands (ARITH 1), but every workgroup quantises the whole input vector of its stage (about 110 lane
// instructions per 8 columns and batch row): at batch 4 that costs as much as the arithmetic saves when a launch
// covers only one layer, and a third less time in long run lists.  Its staging does not depend on the element type,
// so bf16 runs as fast as fp16.  Batch 8 and 16 need more operand columns (batch rows x 3 pieces) than one MFMA has.
// Every workgroup stages the whole input vector of its stage, so larger workgroups mean less staging work per
// row: 1024 lanes everywhere.
#ifndef NQ_STREAM_ARITH
#define NQ_STREAM_ARITH(DT, BATCH) ((BATCH) <= 4 ? 2 : 1)
#endif
#ifndef NQ_STREAM_THREADS
#define NQ_STREAM_THREADS(DT, BATCH) 1024
#endif

// Short lists at batch 4 run faster on the 16-bit arithmetic (its staging is a tenth of the quantising one), long
// ones on the fp4 x fp8 arithmetic: the builder picks per list (`alt`).  At batch 1 and 2 the fp4 x fp8 arithmetic
// wins or ties everywhere.  fp16 only: the 16-bit arithmetic rounds x * s_in and the intermediate vector to the
// activation type, which costs bf16 lists a factor of eight in accuracy (2.3e-3 against 3e-4 of the output maximum)
// where the fp4 x fp8 pieces are as exact for bf16 as for fp16.
constexpr bool stream_alt_exists(int dtype, int batch) { return dtype == 0 && batch == 4; }

template <int DT, int BATCH, int ARITH = NQ_STREAM_ARITH(DT, BATCH)>
struct StreamKernel {
    static constexpr int kArith = ARITH;
    static constexpr int kThreads = NQ_STREAM_THREADS(DT, BATCH);
    static constexpr auto fn = gemv_stream_kernel<DT, BATCH, kArith, kThreads, false, false>;
    static constexpr auto fn_tiled = gemv_stream_kernel<DT, BATCH, kArith, kThreads, false, kArith == 2>;
    // tile order, fp4 x fp8 arithmetic, wavefronts own row pairs: for lists whose longest input is staged in one chunk.
    // It has no row sums in LDS and no LDS atomics, which pays at batch 4 (four batch rows cost four times the flushes)
    // and in long lists at batch 1 and 2; a short slice has fewer row pairs than the workgroup has wavefronts, so the
    // builder asks for it at batch 4 and, for long lists, at batch 1 and 2.
    static constexpr bool kHasOwn = kArith == 2 && BATCH <= 4;
    static constexpr auto fn_tiled_own = gemv_stream_kernel<DT, BATCH, kArith, kThreads, false, kArith == 2, false, kHasOwn>;
    static constexpr auto fn_tiled_own_det = gemv_stream_kernel<DT, BATCH, kArith, kThreads, false, kArith == 2, kHasOwn, kHasOwn>;
    static constexpr auto fn_single = gemv_stream_kernel<DT, BATCH, kArith, kThreads, true, false>;
    // reproducible sums
    // the 16-bit arithmetic is reproducible as it is: the same instance
    static constexpr bool kHasDet = true;
    static constexpr auto fn_det = gemv_stream_kernel<DT, BATCH, kArith, kThreads, false, false, kArith == 2>;
    static constexpr auto fn_tiled_det = gemv_stream_kernel<DT, BATCH, kArith, kThreads, false, kArith == 2, kArith == 2>;
};

template <int DT, int BATCH, int ARITH>
static hipError_t prepare_kernel(size_t lds) {
    using SK = StreamKernel<DT, BATCH, ARITH>;
    static PerDeviceFlag attr_done;              // per template instance and device
    const int dev = current_device();
    if (lds > 64 * 1024 && !attr_done.test(dev)) {
        hipError_t e = hipFuncSetAttribute((const void*)SK::fn,
                                           hipFuncAttributeMaxDynamicSharedMemorySize, kStreamLdsMax);
        if (e != hipSuccess) return e;
        e = hipFuncSetAttribute((const void*)SK::fn_tiled,
                                hipFuncAttributeMaxDynamicSharedMemorySize, kStreamLdsMax);
        if (e != hipSuccess) return e;
        e = hipFuncSetAttribute((const void*)SK::fn_det,
                                hipFuncAttributeMaxDynamicSharedMemorySize, kStreamLdsMax);
        if (e != hipSuccess) return e;
        e = hipFuncSetAttribute((const void*)SK::fn_tiled_det,
                                hipFuncAttributeMaxDynamicSharedMemorySize, kStreamLdsMax);
        if (e != hipSuccess) return e;
        e = hipFuncSetAttribute((const void*)SK::fn_tiled_own,
                                hipFuncAttributeMaxDynamicSharedMemorySize, kStreamLdsMax);
        if (e != hipSuccess) return e;
        e = hipFuncSetAttribute((const void*)SK::fn_tiled_own_det,
                                hipFuncAttributeMaxDynamicSharedMemorySize, kStreamLdsMax);
        if (e != hipSuccess) return e;
        attr_done.set(dev);
    }
    return hipSuccess;
}

// Workgroups of `fn` (launched with `threads` lanes and `lds` bytes of dynamic LDS) that the current device keeps
// resident at once; 0 on error.  The query is host time, so each calling thread keeps its last answers.
static int resident_workgroups(const void* fn, int threads, size_t lds) {
    struct Entry { const void* fn; size_t lds; int dev, cap; };
    static thread_local Entry cache[16];
    static thread_local int used = 0, next = 0;
    const int dev = current_device();
    if (dev < 0) return 0;
    for (int i = 0; i < used; ++i)
        if (cache[i].fn == fn && cache[i].lds == lds && cache[i].dev == dev) return cache[i].cap;
    int per_cu = 0, cus = 0;
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, fn, threads, lds) != hipSuccess) return 0;
    if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) return 0;
    cache[next] = Entry{fn, lds, dev, per_cu * cus};
    next = (next + 1) % 16;
    if (used < 16) ++used;
    return per_cu * cus;
}

// The instance that launch_stream starts for (tiled, det, own) and its LDS plan.  The kernel is only correct when its
// whole grid is resident, so the builder sizes the grid from the smallest capacity over all variants that a plan may
// be launched with (reproducible sums are switched on after the grid is fixed), and launch_stream checks the one
// instance it is about to start.
constexpr int kStreamVariants = 6;      // fn, fn_tiled, fn_det, fn_tiled_det, fn_tiled_own, fn_tiled_own_det
template <int DT, int BATCH, int ARITH>
static const void* stream_variant(int variant, int max_units, int* chunk_cap, size_t* lds) {
    using SK = StreamKernel<DT, BATCH, ARITH>;
    const bool det = variant == 2 || variant == 3 || variant == 5;
    const bool own = variant >= 4;
    if (own && !SK::kHasOwn) return nullptr;
    stream_lds_plan(BATCH, SK::kArith, max_units, chunk_cap, lds, det, own);
    if (own && max_units > *chunk_cap) return nullptr;     // such a list is launched on the row-block form instead
    switch (variant) {
        case 0: return (const void*)SK::fn;
        case 1: return (const void*)SK::fn_tiled;
        case 2: return (const void*)SK::fn_det;
        case 3: return (const void*)SK::fn_tiled_det;
        case 4: return (const void*)SK::fn_tiled_own;
        default: return (const void*)SK::fn_tiled_own_det;
    }
}

// variant < 0: the smallest capacity over all variants; else that of one variant (0: not available or error)
template <int DT, int BATCH, int ARITH>
static int capacity_of(int max_units, int variant = -1) {
    using SK = StreamKernel<DT, BATCH, ARITH>;
    int best = 0;
    for (int v = 0; v < kStreamVariants; ++v) {
        if (variant >= 0 && v != variant) continue;
        int chunk_cap;
        size_t lds;
        const void* fn = stream_variant<DT, BATCH, ARITH>(v, max_units, &chunk_cap, &lds);
        if (!fn) continue;
        if (prepare_kernel<DT, BATCH, ARITH>(lds) != hipSuccess) return 0;
        const int cap = resident_workgroups(fn, SK::kThreads, lds);
        if (cap <= 0) return 0;
        if (best == 0 || cap < best) best = cap;
    }
    return best;
}

template <int DT, int BATCH, int ARITH>
static hipError_t launch_stream(int nstages, const RunSlice* slices, unsigned long long* counters, unsigned* status, int nwg,
                                int max_units, hipStream_t stream, const void* ext_in, void* ext_out, bool tiled, bool det,
                                unsigned spin_limit, bool own) {
    using SK = StreamKernel<DT, BATCH, ARITH>;
    if (spin_limit == 0) spin_limit = 1u << 21;                  // about a second of polling
    if (det && !SK::kHasDet) return hipErrorInvalidValue;
    int chunk_cap;
    size_t lds;
    // the variant whose wavefronts own row pairs, where the plan asks for it and the longest input is one chunk of its
    // (larger) staging area
    own = SK::kHasOwn && own && tiled;
    if (own) {
        stream_lds_plan(BATCH, SK::kArith, max_units, &chunk_cap, &lds, det, true);
        own = max_units <= chunk_cap;
    }
    if (!own) stream_lds_plan(BATCH, SK::kArith, max_units, &chunk_cap, &lds, det);
    hipError_t e = prepare_kernel<DT, BATCH, ARITH>(lds);
    if (e != hipSuccess) return e;
    const bool tiled_fn = tiled && SK::kArith == 2;
    auto fn = own ? (det ? SK::fn_tiled_own_det : SK::fn_tiled_own)
                  : det ? (tiled ? SK::fn_tiled_det : SK::fn_det) : tiled_fn ? SK::fn_tiled : SK::fn;
    // a grid larger than what stays resident would wait for workgroups that never start
    const int cap = resident_workgroups((const void*)fn, SK::kThreads, lds);
    if (cap <= 0) return hipErrorInvalidValue;
    if (nwg > cap) return hipErrorLaunchOutOfResources;
    hipLaunchKernelGGL(fn, dim3(nwg), dim3(SK::kThreads), lds, stream, nstages, slices, counters, status, spin_limit, chunk_cap,
                       RunStage{}, 0, ext_in, ext_out);
    return hipGetLastError();
}

// One stage on its own: the same kernel without tables, dependencies or counters.
template <int DT, int BATCH>
static hipError_t launch_single(const RunStage& st, hipStream_t stream) {
    using SK = StreamKernel<DT, BATCH>;
    int chunk_cap;
    size_t lds;
    stream_lds_plan(BATCH, SK::kArith, st.units, &chunk_cap, &lds);
    static PerDeviceFlag attr_done;              // per template instance and device
    const int dev = current_device();
    if (lds > 64 * 1024 && !attr_done.test(dev)) {
        hipError_t e = hipFuncSetAttribute((const void*)SK::fn_single, hipFuncAttributeMaxDynamicSharedMemorySize, kStreamLdsMax);
        if (e != hipSuccess) return e;
        attr_done.set(dev);
    }
    // resident workgroups of this kernel on this device: the query is host time, so the last answer per calling thread
    // is kept (keyed by device and LDS size)
    static thread_local size_t cached_lds = 0;
    static thread_local int cached_dev = -1, cached_cap = 0;
    if (cached_cap <= 0 || cached_lds != lds || cached_dev != dev) {
        int per_cu = 0, cus = 0;
        if (dev < 0 ||
            hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, (const void*)SK::fn_single, SK::kThreads, lds) != hipSuccess ||
            hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess)
            return hipErrorInvalidValue;
        cached_cap = per_cu * cus;
        cached_lds = lds;
        cached_dev = dev;
    }
    const int cap = cached_cap;
    if (cap <= 0) return hipErrorInvalidValue;
    // whole 16-row groups per workgroup, as few rows as the resident grid allows
    const int rows_per_wg = ((st.rows + cap - 1) / cap + 15) & ~15;
    const int nwg = (st.rows + rows_per_wg - 1) / rows_per_wg;
    hipLaunchKernelGGL((SK::fn_single), dim3(nwg), dim3(SK::kThreads), lds, stream, 0, (const RunSlice*)nullptr,
                       (unsigned long long*)nullptr, (unsigned*)nullptr, 0u, chunk_cap, st, rows_per_wg, (const void*)nullptr,
                       (void*)nullptr);
    return hipGetLastError();
}

// Only the batch sizes that the per-linear path sends here are instantiated.
hipError_t gemv_stream_single(int dtype, int batch, const RunStage& st, hipStream_t stream) {
    if (batch == 8) return dtype == 0 ? launch_single<0, 8>(st, stream) : launch_single<1, 8>(st, stream);
    if (batch != 16) return hipErrorInvalidValue;
    return dtype == 0 ? launch_single<0, 16>(st, stream) : launch_single<1, 16>(st, stream);
}

// CALL(dtype, batch, arithmetic); `alt` selects the 16-bit arithmetic where the batch size has both
#define NQ_STREAM_DISPATCH(CALL)                                                                  \
    if (alt && batch == 4 && dtype == 0) return CALL(0, 4, 1);                                    \
    switch (batch) {                                                                              \
        case 1: return dtype == 0 ? CALL(0, 1, NQ_STREAM_ARITH(0, 1)) : CALL(1, 1, NQ_STREAM_ARITH(1, 1));      \
        case 2: return dtype == 0 ? CALL(0, 2, NQ_STREAM_ARITH(0, 2)) : CALL(1, 2, NQ_STREAM_ARITH(1, 2));      \
        case 4: return dtype == 0 ? CALL(0, 4, NQ_STREAM_ARITH(0, 4)) : CALL(1, 4, NQ_STREAM_ARITH(1, 4));      \
        case 8: return dtype == 0 ? CALL(0, 8, NQ_STREAM_ARITH(0, 8)) : CALL(1, 8, NQ_STREAM_ARITH(1, 8));      \
        case 16: return dtype == 0 ? CALL(0, 16, NQ_STREAM_ARITH(0, 16)) : CALL(1, 16, NQ_STREAM_ARITH(1, 16)); \
        default: break;                                                                           \
    }

// Number of workgroups the device keeps resident for the run-list kernel of this batch size: the smallest over the
// kernel variants a plan may be launched with (variant < 0), or that of one variant (0 on error or where it does not exist).
int stream_capacity(int dtype, int batch, int max_units, bool alt, int variant) {
#define NQ_CAP(D, B, A) capacity_of<D, B, A>(max_units, variant)
    NQ_STREAM_DISPATCH(NQ_CAP)
#undef NQ_CAP
    return 0;
}

// Units of an input vector that are staged at once (longer inputs take several passes over the rows of a slice).
int stream_chunk_cap(int dtype, int batch, int max_units, bool alt) {
    int cap = 0;
    size_t lds = 0;
#define NQ_CHUNK(D, B, A) (stream_lds_plan(B, A, max_units, &cap, &lds), cap)
    NQ_STREAM_DISPATCH(NQ_CHUNK)
#undef NQ_CHUNK
    return 0;
}

// The fp4 x fp8 arithmetic has one kernel per word order: all stages of such a list must agree.
bool stream_needs_uniform_order(int dtype, int batch, bool alt) {
#define NQ_UNI(D, B, A) (A == 2)
    NQ_STREAM_DISPATCH(NQ_UNI)
#undef NQ_UNI
    return false;
}

// Rows that one wave-load spans: slices of tile-order stages are cut at multiples of it.
int stream_row_granule(int dtype, int batch) {
    const bool alt = false;
#define NQ_GRAN(D, B, A) 32
    NQ_STREAM_DISPATCH(NQ_GRAN)
#undef NQ_GRAN
    return 32;
}

// Reproducible sums exist for every batch size that has a run-list kernel.
bool stream_has_deterministic(int dtype, int batch) {
    const bool alt = false;
#define NQ_DET(D, B, A) (StreamKernel<D, B, A>::kHasDet)
    NQ_STREAM_DISPATCH(NQ_DET)
#undef NQ_DET
    return false;
}

hipError_t gemv_stream(int dtype, int batch, int nstages, const RunSlice* slices, unsigned long long* counters,
                       unsigned* status, int nwg, int max_units, hipStream_t stream, const void* ext_in, void* ext_out,
                       bool tiled, bool det, unsigned spin_limit, bool alt, bool own) {
#define NQ_RUN(D, B, A) launch_stream<D, B, A>(nstages, slices, counters, status, nwg, max_units, stream, ext_in, ext_out, tiled, det, spin_limit, own)
    NQ_STREAM_DISPATCH(NQ_RUN)
#undef NQ_RUN
    return hipErrorInvalidValue;
}

bool stream_has_alt(int dtype, int batch) { return stream_alt_exists(dtype, batch); }

}  // namespace nq
