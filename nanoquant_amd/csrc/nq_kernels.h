// Internal launch interface between the C-ABI layer (nq_api.hip) and the kernel files.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace nq {

// nq_gemv.hip: one matmul-free stage.  dtype 0 = fp16, 1 = bf16.  first: input is 16-bit activations
// scaled by s_col; otherwise input is the fp32 intermediate.  Output is fp32 when out_f32, else the
// activation type (clamped); `addend` (fp32, same shape as out) is added before the store.
hipError_t gemv_stage(int dtype, bool first, const uint32_t* bits, const void* in, const void* s_col,
                      const void* s_row, const float* addend, void* out, bool out_f32, int batch, int rows,
                      int words, int K, int in_stride, int out_stride, hipStream_t stream,
                      const void* bias = nullptr);

// Both stages of up to gemv_fused_max() independent linears (batch 1, 2 or 4) in two launches, or in one whose second
// stages wait inside the kernel; see nq_gemv.hip.
int gemv_fused_max();
hipError_t gemv_fused(int dtype, int count, int batch, const void* const* x, const void* const* s_in,
                      const uint32_t* const* vt_bits, const void* const* s_mid, const uint32_t* const* u_bits,
                      const void* const* s_out, const void* const* bias, float* const* h, void* const* y,
                      const int* n, const int* r, const int* m, bool one_launch, hipStream_t stream);
hipError_t gemv_fused_status(unsigned* out, hipStream_t stream);
void gemv_fused_set_spin_limit(unsigned polls);          // 0: the default

// nq_stream.hip: one launch over a table of stages (see the file header).
struct RunStage {
    const uint32_t* bits;   // [rows, words] packed signs, row-major "half2" order
    const void* in;         // [batch, in_stride]: 16-bit activations, or fp32 when in_f32
    const uint16_t* s_col;  // [K] per-column scale applied to a 16-bit input, may be null
    const uint16_t* s_row;  // [rows] per-row scale, may be null
    void* out;              // [batch, out_stride]: fp32 when out_f32, else 16-bit (clamped)
    const float* addend;    // fp32 [batch, out_stride] added before the store, may be null
    const uint16_t* bias;   // [rows] added after the row scale, may be null
    int rows, words, K, units;
    int in_stride, out_stride;
    int in_f32, out_f32;
    int dep, dep2;          // stage indices that must be complete before `in` / `addend` are read, or -1
    int signal;             // a later stage waits on this one
    int vec_bits, vec_in;
    int phase;              // dependency depth: a stage runs after every stage of a lower phase it depends on
    int seg_count;          // number of workgroup slices this stage is cut into (its completion count)
    int in_coherent;        // fp32 input written by another stage of the same launch
    int heavy_release;      // 16-bit output read by a later stage: full device-scope release on completion
    int heavy_acquire;      // 16-bit input written by an earlier stage: full device-scope acquire after the wait
    int tiled;              // `bits` is in the tile order of tile_words() instead of row-major
    int in_ext, out_ext;    // `in` / `out` are given with the launch instead (bound input / output of the list)
    int dep_segs, dep2_segs;  // seg_count of the stages `dep` / `dep2` (what a waiting slice compares the counter with)
    int addend_local;       // the rows of `addend` that a slice reads were written by the slice before it on the same
                            // workgroup (same rows of stage `dep2`): nothing to wait for
};
// One workgroup's share of one stage: rows [row_begin, row_end).
struct RunSegment {
    int stage, row_begin, row_end, pad_;
};
// What the kernel reads per slice, in one record: the slice and a copy of its stage (one dependent memory access
// between the kernel arguments and the first load of data instead of three).  Record w of the table is the first
// slice of workgroup w (stage -1: the workgroup has none); its further slices are the records [more_begin,
// more_end), in the order in which it works them off.
struct RunSlice {
    RunSegment seg;
    int more_begin, more_end;   // meaningful in the first record of a workgroup only
    RunStage st;
};
size_t stream_counter_bytes(int nstages);
// alt: the 16-bit arithmetic instead of the batch size's usual one, where stream_has_alt(dtype, batch);
// own: the fp4 x fp8 kernel whose wavefronts own row pairs, where it exists (tile order, batch 2 and 4, no reproducible
// sums, every input staged in one chunk; ignored otherwise)
int stream_capacity(int dtype, int batch, int max_units, bool alt = false, int variant = -1);
int stream_chunk_cap(int dtype, int batch, int max_units, bool alt = false);
int stream_row_granule(int dtype, int batch);
hipError_t gemv_stream(int dtype, int batch, int nstages, const RunSlice* slices, unsigned long long* counters,
                       unsigned* status, int nwg, int max_units, hipStream_t stream, const void* ext_in = nullptr,
                       void* ext_out = nullptr, bool tiled = false, bool det = false, unsigned spin_limit = 0,
                       bool alt = false, bool own = false);
bool stream_needs_uniform_order(int dtype, int batch, bool alt = false);
bool stream_has_deterministic(int dtype, int batch);
bool stream_has_alt(int dtype, int batch);

// One stage on its own through the run-list kernel (no tables, no counters); batch 16 only.
hipError_t gemv_stream_single(int dtype, int batch, const RunStage& st, hipStream_t stream);

// nq_gemm.hip: C[T,R] = s_out * ((x * s_in) . sgn(W)^T) with W in the 32x256 tile layout.
// scratch: fp32 [T,R] when gemm_scratch_bytes(T,K,R) > 0.
size_t gemm_scratch_bytes(int T, int K, int R);
hipError_t gemm_onebit(int dtype, const void* x, const uint32_t* tiles, const void* s_in, const void* s_out,
                       void* y, float* scratch, int T, int K, int R, hipStream_t stream, const void* bias = nullptr);

// Up to gemm_group_max() GEMMs on the same token count in one launch (s_in: all or none); few-token tiles up to
// gemm_group_max_tokens() tokens, block tiles above.
int gemm_group_max();
int gemm_group_max_tokens();
hipError_t gemm_onebit_group(int dtype, int count, const void* const* x, const uint32_t* const* tiles,
                             const void* const* s_in, const void* const* s_out, const void* const* bias, void* const* y,
                             int T, const int* K, const int* R, hipStream_t stream);

// nq_panel.hip: the same GEMMs at about 128 to 768 tokens as one persistent launch over 64-token x 256-row panels
// (see the file header).  workspace: panel_workspace_bytes() bytes, zero when first used.
size_t panel_workspace_bytes();
bool panel_applies(int count, int T, const int* K, const int* R);
hipError_t gemm_panel_group(int dtype, int count, const void* const* x, const uint32_t* const* tiles,
                            const void* const* s_in, const void* const* s_out, const void* const* bias, void* const* y,
                            int T, const int* K, const int* R, void* workspace, unsigned spin_limit, hipStream_t stream);

// nq_util.hip
hipError_t stream_copy(void* dst, const void* src, size_t bytes, hipStream_t stream);
hipError_t repack_words(const uint32_t* src, uint32_t* dst, size_t nwords, int src_order, int dst_order,
                        hipStream_t stream);
hipError_t words_to_tiles(const uint32_t* src, uint32_t* dst, int rows, int words, int rows_padded, int k_padded,
                          int src_order, hipStream_t stream);
size_t tiled_word_count(int rows, int words);
hipError_t tile_words(const uint32_t* src, uint32_t* dst, int rows, int words, int inverse, hipStream_t stream);

}  // namespace nq
