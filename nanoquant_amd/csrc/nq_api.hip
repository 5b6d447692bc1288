// extern "C" surface of libnq_gfx950.so: argument checks, then kernel launches on the caller's
// stream.  No allocation, no synchronisation, no retained pointers.
#include "../../include/nq_gfx950.h"
#include "nq_kernels.h"

#include <vector>

namespace {
thread_local int g_last_hip_error = 0;

int hip_status(hipError_t e) {
    if (e == hipSuccess) return NQ_OK;
    g_last_hip_error = (int)e;
    (void)hipGetLastError();  // clear the sticky launch error so later calls report their own
    return NQ_ERR_HIP;
}

inline int words_of(int cols) { return (cols + 31) / 32; }
}  // namespace

extern "C" {

const char* nq_status_string(int status) {
    switch (status) {
        case NQ_OK: return "ok";
        case NQ_ERR_DTYPE: return "Support only Half or BFloat16";
        case NQ_ERR_NULL: return "required pointer is null";
        case NQ_ERR_SHAPE: return "invalid or inconsistent sizes";
        case NQ_ERR_K_MISMATCH: return "k dimension mismatch";
        case NQ_ERR_PROB_SHAPE: return "Problem shape incompatible";
        case NQ_ERR_WORKSPACE: return "workspace too small";
        case NQ_ERR_ORDER: return "unknown word order";
        case NQ_ERR_ALIGN: return "prefill operands must be 16-byte aligned";
        case NQ_ERR_HIP: return "HIP runtime error";
        default: return "unknown status";
    }
}

int nq_last_hip_error(void) { return g_last_hip_error; }

int nq_abi_version(void) { return 1; }

int nq_device_query(int attr, int* value) {
    if (!value) return NQ_ERR_NULL;
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return hip_status(e);
    hipDeviceAttribute_t which;
    switch (attr) {
        case NQ_ATTR_CU_COUNT: which = hipDeviceAttributeMultiprocessorCount; break;
        case NQ_ATTR_LDS_BYTES: which = hipDeviceAttributeMaxSharedMemoryPerBlock; break;
        case NQ_ATTR_WAVE_SIZE: which = hipDeviceAttributeWarpSize; break;
        default: return NQ_ERR_SHAPE;
    }
    return hip_status(hipDeviceGetAttribute(value, which, dev));
}

int nq_gemv_forward(const void* x, const void* s_in, const uint32_t* vt_bits, const void* s_mid,
                    const uint32_t* u_bits, const void* s_out, float* h_scratch, void* y,
                    int batch, int n, int r, int m, int dtype, void* stream) {
    if (dtype != NQ_F16 && dtype != NQ_BF16) return NQ_ERR_DTYPE;
    if (batch < 0 || n < 0 || r < 0 || m < 0) return NQ_ERR_SHAPE;
    if (batch == 0 || m == 0) return NQ_OK;
    if (!x || !s_in || !vt_bits || !u_bits || !s_out || !h_scratch || !y) return NQ_ERR_NULL;
    hipStream_t st = (hipStream_t)stream;
    hipError_t e = nq::gemv_stage(dtype, true, vt_bits, x, s_in, s_mid, nullptr, h_scratch, true, batch, r,
                                  words_of(n), n, n, r, st);
    if (e != hipSuccess) return hip_status(e);
    e = nq::gemv_stage(dtype, false, u_bits, h_scratch, nullptr, s_out, nullptr, y, false, batch, m,
                       words_of(r), r, r, m, st);
    return hip_status(e);
}

int nq_gemv_mixture(const void* x, const void* const* s_in, const uint32_t* const* vt_bits,
                    const void* const* s_mid, const uint32_t* const* u_bits, const void* const* s_out,
                    const int* r, int nterms, float* h_scratch, float* y_scratch, void* y,
                    int batch, int n, int m, int dtype, void* stream) {
    if (dtype != NQ_F16 && dtype != NQ_BF16) return NQ_ERR_DTYPE;
    if (batch < 0 || n < 0 || m < 0 || nterms < 1) return NQ_ERR_SHAPE;
    if (!x || !s_in || !vt_bits || !s_mid || !u_bits || !s_out || !r || !h_scratch || !y) return NQ_ERR_NULL;
    if (nterms > 1 && !y_scratch) return NQ_ERR_NULL;
    for (int t = 0; t < nterms; ++t) {
        if (r[t] < 0) return NQ_ERR_SHAPE;
        if (!s_in[t] || !vt_bits[t] || !u_bits[t] || !s_out[t]) return NQ_ERR_NULL;
    }
    if (batch == 0 || m == 0) return NQ_OK;
    hipStream_t st = (hipStream_t)stream;
    for (int t = 0; t < nterms; ++t) {
        hipError_t e = nq::gemv_stage(dtype, true, vt_bits[t], x, s_in[t], s_mid[t], nullptr, h_scratch, true,
                                      batch, r[t], words_of(n), n, n, r[t], st);
        if (e != hipSuccess) return hip_status(e);
        const bool last = (t == nterms - 1);
        // Partial sums over terms stay in fp32; only the last term rounds to the activation type.
        e = nq::gemv_stage(dtype, false, u_bits[t], h_scratch, nullptr, s_out[t], t ? y_scratch : nullptr,
                           last ? y : (void*)y_scratch, !last, batch, m, words_of(r[t]), r[t], r[t], m, st);
        if (e != hipSuccess) return hip_status(e);
    }
    return NQ_OK;
}

int nq_gemv_stage(const void* in, const void* s_col, const uint32_t* bits, const void* s_row, void* out,
                  int batch, int cols, int rows, int dtype, void* stream) {
    if (dtype != NQ_F16 && dtype != NQ_BF16) return NQ_ERR_DTYPE;
    if (batch < 0 || cols < 0 || rows < 0) return NQ_ERR_SHAPE;
    if (batch == 0 || rows == 0) return NQ_OK;
    if (!in || !bits || !out) return NQ_ERR_NULL;
    return hip_status(nq::gemv_stage(dtype, true, bits, in, s_col, s_row, nullptr, out, false, batch, rows,
                                     words_of(cols), cols, cols, rows, (hipStream_t)stream));
}

// ---- run list ---------------------------------------------------------------------------------
// workspace layout: [0,256): status word; counters (one per stage + the exit counter, rounded to
// 256 bytes); 2n RunStage records (rounded to 256 bytes); one int per workgroup naming its stage.
static size_t round256(size_t v) { return (v + 255) / 256 * 256; }
static size_t runlist_counter_bytes(int n) { return round256(nq::stream_counter_bytes(2 * n)); }
static size_t runlist_table_bytes(int n) { return round256((size_t)2 * n * sizeof(nq::RunStage)); }

static int stage_workgroups(int rows, int cols) {
    const int units = ((cols + 31) / 32 + 3) / 4;
    const int per = nq::stream_rows_per_item(units);
    return (rows + per - 1) / per;
}

size_t nq_runlist_workspace_bytes(const nq_linear* linears, int nlinears) {
    if (nlinears <= 0 || !linears) return 0;
    size_t wgs = 0;
    for (int i = 0; i < nlinears; ++i) {
        if (linears[i].n <= 0 || linears[i].r <= 0 || linears[i].m <= 0) return 0;
        wgs += (size_t)stage_workgroups(linears[i].r, linears[i].n) + (size_t)stage_workgroups(linears[i].m, linears[i].r);
    }
    return 256 + runlist_counter_bytes(nlinears) + runlist_table_bytes(nlinears) + round256(wgs * sizeof(int));
}

static inline bool al16(const void* p) { return ((uintptr_t)p & 15u) == 0; }

int nq_runlist_build(const nq_linear* linears, int nlinears, int batch, int dtype, int interleave,
                     void* workspace, size_t workspace_bytes, nq_runlist_plan* plan_out, void* stream) {
    if (!plan_out) return NQ_ERR_NULL;
    if (dtype != NQ_F16 && dtype != NQ_BF16) return NQ_ERR_DTYPE;
    if (nlinears <= 0 || interleave < 1) return NQ_ERR_SHAPE;
    if (batch != 1 && batch != 2 && batch != 4 && batch != 8 && batch != 16) return NQ_ERR_SHAPE;
    if (!linears || !workspace) return NQ_ERR_NULL;
    if (((uintptr_t)workspace & 255u) != 0) return NQ_ERR_ALIGN;
    for (int i = 0; i < nlinears; ++i) {
        const nq_linear& l = linears[i];
        if (l.n <= 0 || l.r <= 0 || l.m <= 0) return NQ_ERR_SHAPE;
        if (!l.x || !l.s_in || !l.vt_bits || !l.u_bits || !l.s_out || !l.h || !l.y) return NQ_ERR_NULL;
        if (l.x_from >= i || l.y_from >= i) return NQ_ERR_SHAPE;
        if (l.y_from >= 0 && !linears[l.y_from].out_f32) return NQ_ERR_SHAPE;   // addends are fp32 results
    }
    if (workspace_bytes < nq_runlist_workspace_bytes(linears, nlinears)) return NQ_ERR_WORKSPACE;
    // Order of stages: first stages run ahead of second stages by up to `interleave` linears, unless a
    // dependency (or a shared h buffer) forces a second stage out earlier.
    std::vector<nq::RunStage> table;
    std::vector<int> first_idx(nlinears, -1), second_idx(nlinears, -1);
    std::vector<int> pending;
    auto emit_second = [&](int i) {
        const nq_linear& l = linears[i];
        nq::RunStage st{};
        st.bits = l.u_bits; st.in = l.h; st.s_col = nullptr; st.s_row = (const uint16_t*)l.s_out;
        st.out = l.y; st.addend = l.addend;
        st.rows = l.m; st.K = l.r; st.words = (l.r + 31) / 32; st.units = (st.words + 3) / 4;
        st.in_stride = l.r; st.out_stride = l.m; st.in_f32 = 1; st.out_f32 = l.out_f32 ? 1 : 0;
        st.dep = first_idx[i];
        st.in_coherent = 1;
        st.dep2 = (l.addend && l.y_from >= 0) ? second_idx[l.y_from] : -1;
        st.signal = 0;
        st.vec_bits = (st.words % 4 == 0) && al16(l.u_bits);
        st.vec_in = al16(l.h) && ((size_t)l.r * 4) % 16 == 0;
        second_idx[i] = (int)table.size();
        table.push_back(st);
    };
    auto flush_until = [&](int upto_linear) {   // emit pending second stages in order up to `upto_linear`
        while (!pending.empty()) {
            const int i = pending.front();
            emit_second(i);
            pending.erase(pending.begin());
            if (i == upto_linear) break;
        }
    };
    for (int i = 0; i < nlinears; ++i) {
        const nq_linear& l = linears[i];
        int need = -1;
        for (int j : pending) {
            if (j == l.x_from || j == l.y_from || linears[j].h == l.h) need = j;
        }
        if (need >= 0) flush_until(need);
        nq::RunStage st{};
        st.bits = l.vt_bits; st.in = l.x; st.s_col = (const uint16_t*)l.s_in; st.s_row = (const uint16_t*)l.s_mid;
        st.out = l.h; st.addend = nullptr;
        st.rows = l.r; st.K = l.n; st.words = (l.n + 31) / 32; st.units = (st.words + 3) / 4;
        st.in_stride = l.n; st.out_stride = l.r; st.in_f32 = 0; st.out_f32 = 1;
        st.dep = l.x_from >= 0 ? second_idx[l.x_from] : -1;
        if (st.dep >= 0) {                       // 16-bit y of an earlier linear is this linear's x
            st.heavy_acquire = 1;
            table[st.dep].heavy_release = 1;
        }
        st.dep2 = -1;
        st.signal = 0;
        st.vec_bits = (st.words % 4 == 0) && al16(l.vt_bits);
        st.vec_in = al16(l.x) && ((size_t)l.n * 2) % 16 == 0 && al16(l.s_in);
        first_idx[i] = (int)table.size();
        table.push_back(st);
        pending.push_back(i);
        if ((int)pending.size() >= interleave) flush_until(pending.front());
    }
    flush_until(-1);
    for (auto& st : table) st.signal = 0;
    int total_wgs = 0, max_units = 1;
    for (auto& st : table) {
        if (st.units > max_units) max_units = st.units;
        if (st.dep >= 0) table[st.dep].signal = 1;
        if (st.dep2 >= 0) table[st.dep2].signal = 1;
        st.rows_item = nq::stream_rows_per_item(st.units);
        st.wg_begin = total_wgs;
        st.wg_count = (st.rows + st.rows_item - 1) / st.rows_item;
        total_wgs += st.wg_count;
    }
    std::vector<int> wg_stage((size_t)total_wgs);
    for (size_t si = 0; si < table.size(); ++si)
        for (int w = 0; w < table[si].wg_count; ++w) wg_stage[(size_t)table[si].wg_begin + w] = (int)si;
    hipStream_t hs = (hipStream_t)stream;
    char* base = (char*)workspace;
    const size_t off_table = 256 + runlist_counter_bytes(nlinears);
    const size_t off_map = off_table + runlist_table_bytes(nlinears);
    hipError_t e = hipMemsetAsync(base, 0, off_table, hs);
    if (e != hipSuccess) return hip_status(e);
    e = hipMemcpyAsync(base + off_table, table.data(), table.size() * sizeof(nq::RunStage), hipMemcpyHostToDevice, hs);
    if (e != hipSuccess) return hip_status(e);
    e = hipMemcpyAsync(base + off_map, wg_stage.data(), wg_stage.size() * sizeof(int), hipMemcpyHostToDevice, hs);
    if (e != hipSuccess) return hip_status(e);
    plan_out->nlinears = nlinears;
    plan_out->nstages = (int)table.size();
    plan_out->total_workgroups = total_wgs;
    plan_out->max_units = max_units;
    plan_out->batch = batch;
    plan_out->dtype = dtype;
    return hip_status(hipStreamSynchronize(hs));   // `table` is host memory: finish before it dies
}

int nq_runlist_run(const void* workspace, const nq_runlist_plan* plan, void* stream) {
    if (!workspace || !plan) return NQ_ERR_NULL;
    if (plan->dtype != NQ_F16 && plan->dtype != NQ_BF16) return NQ_ERR_DTYPE;
    if (plan->nlinears <= 0 || plan->nstages != 2 * plan->nlinears || plan->total_workgroups <= 0 ||
        plan->max_units <= 0)
        return NQ_ERR_SHAPE;
    const int batch = plan->batch;
    if (batch != 1 && batch != 2 && batch != 4 && batch != 8 && batch != 16) return NQ_ERR_SHAPE;
    char* base = (char*)workspace;
    const size_t off_table = 256 + runlist_counter_bytes(plan->nlinears);
    const size_t off_map = off_table + runlist_table_bytes(plan->nlinears);
    return hip_status(nq::gemv_stream(plan->dtype, batch, (const nq::RunStage*)(base + off_table), plan->nstages,
                                      (const int*)(base + off_map), (unsigned long long*)(base + 256), (unsigned*)base,
                                      plan->total_workgroups, plan->max_units, (hipStream_t)stream));
}

int nq_runlist_status(const void* workspace, int* status_out, void* stream) {
    if (!workspace || !status_out) return NQ_ERR_NULL;
    unsigned v = 0;
    hipError_t e = hipMemcpyAsync(&v, workspace, sizeof(v), hipMemcpyDeviceToHost, (hipStream_t)stream);
    if (e != hipSuccess) return hip_status(e);
    e = hipStreamSynchronize((hipStream_t)stream);
    *status_out = (int)v;
    return hip_status(e);
}

size_t nq_gemm_scratch_bytes(int tokens, int k, int rows) { return nq::gemm_scratch_bytes(tokens, k, rows); }

int nq_gemm_onebit(const void* x, const uint32_t* tiles, const void* s_in, const void* s_out, void* y,
                   void* scratch, size_t scratch_bytes, int tokens, int k, int rows, int dtype, void* stream) {
    if (dtype != NQ_F16 && dtype != NQ_BF16) return NQ_ERR_DTYPE;
    if (tokens < 0 || k < 0 || rows < 0) return NQ_ERR_SHAPE;
    if (k % 256 != 0 || rows % 32 != 0) return NQ_ERR_PROB_SHAPE;
    if (tokens == 0 || rows == 0 || k == 0) return NQ_OK;
    if (!x || !tiles || !y) return NQ_ERR_NULL;
    if (((uintptr_t)x | (uintptr_t)tiles | (uintptr_t)y | (uintptr_t)s_in | (uintptr_t)scratch) & 15u) return NQ_ERR_ALIGN;
    const size_t need = nq::gemm_scratch_bytes(tokens, k, rows);
    if (need > 0 && (!scratch || scratch_bytes < need)) return NQ_ERR_WORKSPACE;
    return hip_status(nq::gemm_onebit(dtype, x, tiles, s_in, s_out, y, (float*)scratch, tokens, k, rows,
                                      (hipStream_t)stream));
}

int nq_gemm_nanoquant(const void* x, const uint32_t* vt_tiles, const uint32_t* u_tiles, const void* s_in,
                      const void* s_mid, const void* s_out, void* h, void* y, void* scratch,
                      size_t scratch_bytes, int tokens, int n, int r, int m, int dtype, void* stream) {
    if (!h) return (tokens == 0 || m == 0) ? NQ_OK : NQ_ERR_NULL;
    int st = nq_gemm_onebit(x, vt_tiles, s_in, s_mid, h, scratch, scratch_bytes, tokens, n, r, dtype, stream);
    if (st != NQ_OK) return st;
    return nq_gemm_onebit(h, u_tiles, nullptr, s_out, y, scratch, scratch_bytes, tokens, r, m, dtype, stream);
}

int nq_repack_words(const uint32_t* src, uint32_t* dst, size_t nwords, int src_order, int dst_order, void* stream) {
    if ((src_order != 0 && src_order != 1) || (dst_order != 0 && dst_order != 1)) return NQ_ERR_ORDER;
    if (nwords == 0) return NQ_OK;
    if (!src || !dst) return NQ_ERR_NULL;
    return hip_status(nq::repack_words(src, dst, nwords, src_order, dst_order, (hipStream_t)stream));
}

int nq_stream_copy(void* dst, const void* src, size_t bytes, void* stream) {
    if (bytes % 16 != 0) return NQ_ERR_SHAPE;
    if (bytes == 0) return NQ_OK;
    if (!src || !dst) return NQ_ERR_NULL;
    return hip_status(nq::stream_copy(dst, src, bytes, (hipStream_t)stream));
}

}  // extern "C"
