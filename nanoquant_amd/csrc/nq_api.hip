// extern "C" surface of libnq_gfx950.so: argument checks, then kernel launches on the caller's
// stream.  No allocation, no synchronisation, no retained pointers.
#include "../../include/nq_gfx950.h"
#include "nq_kernels.h"

#include <algorithm>
#include <atomic>
#include <mutex>
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
        case NQ_ERR_SCRATCH_LIMIT: return "batch * r exceeds the built-in scratch of the allocation-free entry point";
        case NQ_ERR_HIP: return "HIP runtime error";
        default: return "unknown status";
    }
}

int nq_last_hip_error(void) { return g_last_hip_error; }

int nq_abi_version(void) { return 9; }

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
    return nq_gemv_forward_bias(x, s_in, vt_bits, s_mid, u_bits, s_out, nullptr, h_scratch, y, batch, n, r, m, dtype, stream);
}

// Both stages of every linear for `batch` rows.  Groups of independent linears in pieces of 1, 2 and 4 batch rows go
// through nq::gemv_fused (two launches per nq::gemv_fused_max() linears, or one with `one_launch`); a single linear,
// and pieces of 8 and 16 rows, take two launches per linear.
static int forward_linears(const nq_linear* ls, int count, int batch, int dtype, bool one_launch, hipStream_t st) {
    const int group = nq::gemv_fused_max();
    int done = 0;
    while (done < batch) {
        int piece = 16;
        while (piece > batch - done) piece >>= 1;
        if (piece >= 8 || (count == 1 && !one_launch)) {
            for (int i = 0; i < count; ++i) {
                const nq_linear& l = ls[i];
                if (l.m == 0) continue;
                const char* x = (const char*)l.x + (size_t)done * l.n * 2;
                float* h = l.h + (size_t)done * l.r;
                char* y = (char*)l.y + (size_t)done * l.m * 2;
                hipError_t e = nq::gemv_stage(dtype, true, l.vt_bits, x, l.s_in, l.s_mid, nullptr, h, true, piece, l.r,
                                              words_of(l.n), l.n, l.n, l.r, st);
                if (e != hipSuccess) return hip_status(e);
                e = nq::gemv_stage(dtype, false, l.u_bits, h, nullptr, l.s_out, nullptr, y, false, piece, l.m,
                                   words_of(l.r), l.r, l.r, l.m, st, l.bias);
                if (e != hipSuccess) return hip_status(e);
            }
        } else {
            for (int i0 = 0; i0 < count; i0 += group) {
                const int c = count - i0 < group ? count - i0 : group;
                const void *x[16], *s_in[16], *s_mid[16], *s_out[16], *bias[16];
                const uint32_t *vt[16], *u[16];
                float* h[16];
                void* y[16];
                int n[16], r[16], m[16];
                int k = 0;
                for (int i = i0; i < i0 + c; ++i) {
                    const nq_linear& l = ls[i];
                    if (l.m == 0) continue;
                    x[k] = (const char*)l.x + (size_t)done * l.n * 2;
                    h[k] = l.h + (size_t)done * l.r;
                    y[k] = (char*)l.y + (size_t)done * l.m * 2;
                    s_in[k] = l.s_in; s_mid[k] = l.s_mid; s_out[k] = l.s_out; bias[k] = l.bias;
                    vt[k] = l.vt_bits; u[k] = l.u_bits;
                    n[k] = l.n; r[k] = l.r; m[k] = l.m;
                    ++k;
                }
                if (k == 0) continue;
                hipError_t e = nq::gemv_fused(dtype, k, piece, x, s_in, vt, s_mid, u, s_out, bias, h, y, n, r, m, one_launch, st);
                if (e != hipSuccess) return hip_status(e);
            }
        }
        done += piece;
    }
    return NQ_OK;
}

int nq_gemv_forward_bias(const void* x, const void* s_in, const uint32_t* vt_bits, const void* s_mid,
                         const uint32_t* u_bits, const void* s_out, const void* bias, float* h_scratch, void* y,
                         int batch, int n, int r, int m, int dtype, void* stream) {
    if (dtype != NQ_F16 && dtype != NQ_BF16) return NQ_ERR_DTYPE;
    if (batch < 0 || n < 0 || r < 0 || m < 0) return NQ_ERR_SHAPE;
    if (batch == 0 || m == 0) return NQ_OK;
    if (!x || !s_in || !vt_bits || !u_bits || !s_out || !h_scratch || !y) return NQ_ERR_NULL;
    nq_linear l{};
    l.x = x; l.s_in = s_in; l.vt_bits = vt_bits; l.s_mid = s_mid; l.u_bits = u_bits; l.s_out = s_out;
    l.h = h_scratch; l.y = y; l.bias = bias; l.n = n; l.r = r; l.m = m; l.x_from = -1; l.y_from = -1;
    return forward_linears(&l, 1, batch, dtype, false, (hipStream_t)stream);
}

int nq_gemv_group_max(void) { return nq::gemv_fused_max(); }

int nq_gemv_forward_group(const nq_linear* linears, int count, int batch, int dtype, int one_launch, void* stream) {
    if (dtype != NQ_F16 && dtype != NQ_BF16) return NQ_ERR_DTYPE;
    if (count < 0 || batch < 0 || (one_launch != 0 && one_launch != 1)) return NQ_ERR_SHAPE;
    if (count == 0 || batch == 0) return NQ_OK;
    if (!linears) return NQ_ERR_NULL;
    for (int i = 0; i < count; ++i) {
        const nq_linear& l = linears[i];
        if (l.n < 0 || l.r < 0 || l.m < 0) return NQ_ERR_SHAPE;
        if (l.x_from >= 0 || l.y_from >= 0 || l.addend || l.out_f32 || l.tiled) return NQ_ERR_SHAPE;   // independent plain linears only
        if (l.m == 0) continue;
        if (!l.x || !l.s_in || !l.vt_bits || !l.u_bits || !l.s_out || !l.h || !l.y) return NQ_ERR_NULL;
        for (int j = 0; j < i; ++j)
            if (linears[j].m && linears[j].h == l.h) return NQ_ERR_SHAPE;                               // every linear needs an h of its own
    }
    return forward_linears(linears, count, batch, dtype, one_launch != 0, (hipStream_t)stream);
}

int nq_gemv_group_set_spin_limit(unsigned polls) {
    nq::gemv_fused_set_spin_limit(polls);
    return NQ_OK;
}

int nq_gemv_group_status(int* status_out, void* stream) {
    if (!status_out) return NQ_ERR_NULL;
    unsigned v = 0;
    hipError_t e = nq::gemv_fused_status(&v, (hipStream_t)stream);
    if (e != hipSuccess) return hip_status(e);
    *status_out = (int)v;
    return NQ_OK;
}

// ---- the allocation-free variant of nq_gemv_forward_bias ---------------------------------------------
// The fp32 intermediate h lives in a file-scope device array instead of a caller's buffer.  In host code the
// array's name is only a handle: its device address is asked for once per device (each device holds its own copy)
// and only that address is ever handed to a kernel.
constexpr size_t kScratchFloats = NQ_NOALLOC_MAX_H_FLOATS;
static __device__ __align__(256) float scratch[kScratchFloats];
constexpr int kScratchMaxDevices = 64;
static float* g_scratch_ptr[kScratchMaxDevices];
static std::mutex g_scratch_mutex;

static int scratch_address(float** out) {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return hip_status(e);
    if (dev < 0 || dev >= kScratchMaxDevices) return NQ_ERR_SHAPE;
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        float* p = nullptr;
        e = hipGetSymbolAddress((void**)&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess) return hip_status(e);
        if (!p) return NQ_ERR_NULL;
        g_scratch_ptr[dev] = p;
    }
    *out = g_scratch_ptr[dev];
    return NQ_OK;
}

int nq_gemv_forward_noalloc(const void* x, const void* s_in, const uint32_t* vt_bits, const void* s_mid,
                            const uint32_t* u_bits, const void* s_out, const void* bias, void* y,
                            int batch, int n, int r, int m, int dtype, void* stream) {
    if (dtype != NQ_F16 && dtype != NQ_BF16) return NQ_ERR_DTYPE;
    if (batch < 0 || n < 0 || r < 0 || m < 0) return NQ_ERR_SHAPE;
    if ((unsigned long long)batch * (unsigned long long)r > kScratchFloats) return NQ_ERR_SCRATCH_LIMIT;
    if (batch == 0 || m == 0) return NQ_OK;
    if (!x || !s_in || !vt_bits || !u_bits || !s_out || !y) return NQ_ERR_NULL;
    float* h = nullptr;
    const int st = scratch_address(&h);
    if (st != NQ_OK) return st;
    return nq_gemv_forward_bias(x, s_in, vt_bits, s_mid, u_bits, s_out, bias, h, y, batch, n, r, m, dtype, stream);
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
// workspace layout: [0,256): status word; completion counters; the slice records (each with a copy of its stage).
// Every block is rounded to 256 bytes.
static size_t round256(size_t v) { return (v + 255) / 256 * 256; }
static size_t runlist_counter_bytes(int n) { return round256(nq::stream_counter_bytes(2 * n)); }
constexpr int kMaxResidentWorkgroups = 1024;   // upper bound used for sizing only (1024-lane workgroups: 1-2 per CU)

// slices: one first record per workgroup, then at most one more per workgroup and phase and one per stage
static size_t runlist_slice_bytes(int nwg, int nphases, int nstages) {
    return round256(((size_t)nwg * (nphases + 1) + nstages) * sizeof(nq::RunSlice));
}

size_t nq_runlist_workspace_bytes(const nq_linear* linears, int nlinears) {
    if (nlinears <= 0 || !linears) return 0;
    // phases <= stages; a generous bound keeps the call independent of the device
    int depth_bound = 2;
    for (int i = 0; i < nlinears; ++i)
        if (linears[i].x_from >= 0 || linears[i].y_from >= 0) depth_bound += 2;
    if (depth_bound > 2 * nlinears) depth_bound = 2 * nlinears;
    return 256 + runlist_counter_bytes(nlinears) + runlist_slice_bytes(kMaxResidentWorkgroups, depth_bound, 2 * nlinears);
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
        if (!l.s_in || !l.vt_bits || !l.u_bits || !l.s_out || !l.h) return NQ_ERR_NULL;   // x, y NULL: bound at run time
        if (!l.x && l.x_from >= 0) return NQ_ERR_SHAPE;
        if (l.x_from >= i || l.y_from >= i) return NQ_ERR_SHAPE;
        if (l.x_from >= 0 && !linears[l.x_from].y) return NQ_ERR_SHAPE;   // a bound output cannot feed another entry
        if (l.y_from >= 0 && !linears[l.y_from].y) return NQ_ERR_SHAPE;
        if (l.y_from >= 0 && !linears[l.y_from].out_f32) return NQ_ERR_SHAPE;   // addends are fp32 results
        // a link must name the buffer, width and type that the earlier entry really produces: the kernel reads
        // x as [batch, n] of the 16-bit type and the addend as fp32 [batch, m]
        if (l.x_from >= 0) {
            const nq_linear& p = linears[l.x_from];
            if (l.x != p.y || l.n != p.m || p.out_f32) return NQ_ERR_SHAPE;
        }
        if (l.y_from >= 0) {
            const nq_linear& p = linears[l.y_from];
            if (l.addend != (const float*)p.y || l.m != p.m) return NQ_ERR_SHAPE;
        }
        // two linears writing the same h would race inside a phase
        for (int j = 0; j < i; ++j)
            if (linears[j].h == l.h) return NQ_ERR_SHAPE;
    }
    if (nq::stream_needs_uniform_order(dtype, batch))       // one kernel per word order at these batch sizes
        for (int i = 1; i < nlinears; ++i)
            if ((linears[i].tiled != 0) != (linears[0].tiled != 0)) return NQ_ERR_SHAPE;
    int bound_n = 0, bound_outputs = 0;
    for (int i = 0; i < nlinears; ++i) {         // one bound x (shared by every entry that reads it), one bound y
        if (!linears[i].x) {
            if (bound_n && bound_n != linears[i].n) return NQ_ERR_SHAPE;
            bound_n = linears[i].n;
        }
        if (!linears[i].y && ++bound_outputs > 1) return NQ_ERR_SHAPE;
    }
    if (workspace_bytes < nq_runlist_workspace_bytes(linears, nlinears)) return NQ_ERR_WORKSPACE;
    (void)interleave;   // kept for interface stability: phases make the ordering hint unnecessary

    // ---- stage table: stage 2i = first stage of linear i, 2i+1 = its second stage -------------------
    const int nstages = 2 * nlinears;
    std::vector<nq::RunStage> table((size_t)nstages);
    int max_units = 1, nphases = 0;
    for (int i = 0; i < nlinears; ++i) {
        const nq_linear& l = linears[i];
        nq::RunStage a{};
        a.bits = l.vt_bits; a.in = l.x; a.s_col = (const uint16_t*)l.s_in; a.s_row = (const uint16_t*)l.s_mid;
        a.out = l.h; a.addend = nullptr; a.tiled = l.tiled ? 1 : 0; a.in_ext = l.x ? 0 : 1;
        a.rows = l.r; a.K = l.n; a.words = (l.n + 31) / 32; a.units = (a.words + 3) / 4;
        a.in_stride = l.n; a.out_stride = l.r; a.in_f32 = 0; a.out_f32 = 1;
        a.dep = l.x_from >= 0 ? 2 * l.x_from + 1 : -1;
        a.dep2 = -1;
        a.vec_bits = (a.words % 4 == 0) && al16(l.vt_bits);
        a.vec_in = al16(l.x) && ((size_t)l.n * 2) % 16 == 0 && al16(l.s_in);   // a bound x must be 16-byte aligned
        a.phase = a.dep >= 0 ? table[a.dep].phase + 1 : 0;
        if (a.dep >= 0) {                        // 16-bit y of an earlier linear is this linear's x
            a.heavy_acquire = 1;
            table[a.dep].heavy_release = 1;
        }
        table[2 * i] = a;

        nq::RunStage b{};
        b.bits = l.u_bits; b.in = l.h; b.s_col = nullptr; b.s_row = (const uint16_t*)l.s_out;
        b.out = l.y; b.addend = l.addend; b.bias = (const uint16_t*)l.bias; b.tiled = l.tiled ? 1 : 0; b.out_ext = l.y ? 0 : 1;
        b.rows = l.m; b.K = l.r; b.words = (l.r + 31) / 32; b.units = (b.words + 3) / 4;
        b.in_stride = l.r; b.out_stride = l.m; b.in_f32 = 1; b.out_f32 = l.out_f32 ? 1 : 0;
        b.dep = 2 * i;
        b.in_coherent = 1;
        b.dep2 = (l.addend && l.y_from >= 0) ? 2 * l.y_from + 1 : -1;
        b.vec_bits = (b.words % 4 == 0) && al16(l.u_bits);
        b.vec_in = al16(l.h) && ((size_t)l.r * 4) % 16 == 0;
        b.phase = a.phase + 1;
        if (b.dep2 >= 0) {
            // A term that adds onto the result of an earlier one: where its own input is ready in time, it runs in the
            // phase of that stage, cut into the same rows on the same workgroups, each slice right behind the one that
            // writes its addend -- nothing to wait for between the two.  Otherwise it runs a phase later and waits
            // for the whole earlier stage.
            const nq::RunStage& head = table[b.dep2];
            if (a.phase + 1 <= head.phase && (head.tiled != 0) == (l.tiled != 0)) {
                b.phase = head.phase;
                b.addend_local = 1;
            } else if (head.phase + 1 > b.phase) {
                b.phase = head.phase + 1;
            }
        }
        // the kernel addresses the packed words of a stage with 32-bit byte offsets
        const size_t bytes_a = l.tiled ? nq::tiled_word_count(a.rows, a.words) * 4 : (size_t)a.rows * a.words * 4;
        const size_t bytes_b = l.tiled ? nq::tiled_word_count(b.rows, b.words) * 4 : (size_t)b.rows * b.words * 4;
        if (bytes_a >= 0x7FFFFFF0ull || bytes_b >= 0x7FFFFFF0ull) return NQ_ERR_SHAPE;
        if (l.tiled && (((uintptr_t)l.vt_bits | (uintptr_t)l.u_bits) & 15u)) return NQ_ERR_ALIGN;
        table[2 * i + 1] = b;
        if (a.units > max_units) max_units = a.units;
        if (b.units > max_units) max_units = b.units;
        if (b.phase + 1 > nphases) nphases = b.phase + 1;
    }
    for (auto& st : table) {
        if (st.dep >= 0) table[st.dep].signal = 1;
        if (st.dep2 >= 0) table[st.dep2].signal = 1;
    }

    // ---- grid = what the device keeps resident; every workgroup gets an equal share of every phase ----
    // Which arithmetic: at batch 4 (fp16) a list with little work per workgroup (up to two Llama-2-7B layers on 256
    // workgroups: 14000 rows x 16-byte units each) runs on the 16-bit arithmetic of batch 8 and 16, whose staging costs a
    // tenth of the quantising one; longer lists stream faster on the fp4 x fp8 arithmetic (the two cross at 2.6 layers).
    bool alt = false;
    if (nq::stream_has_alt(dtype, batch)) {
        long long work = 0;
        for (const auto& st : table) work += (long long)st.rows * st.units;
        const int usual = nq::stream_capacity(dtype, batch, max_units, false);
        if (usual <= 0) return NQ_ERR_HIP;
        alt = work / usual <= 14000;
    }
    const bool wide = batch >= 8 || alt;                 // the 16-bit arithmetic and its cost model
    // fp4 x fp8 arithmetic with wavefronts that own row pairs (tile order only; the launch falls back where it does not
    // apply): always at batch 4, from about six Llama-2-7B layers per launch on at batch 1 and 2 (40000 rows x units per
    // workgroup), where a slice has more row pairs than the workgroup has wavefronts
    bool own = false;
    if (!alt && batch <= 4) {
        long long work = 0;
        for (const auto& st : table) work += (long long)st.rows * st.units;
        own = batch == 4 || work / std::max(1, nq::stream_capacity(dtype, batch, max_units, false)) >= 40000;
    }
    const int granule = nq::stream_row_granule(dtype, batch);
    int nwg = nq::stream_capacity(dtype, batch, max_units, alt);
    if (nwg <= 0) return NQ_ERR_HIP;
    if (nwg > kMaxResidentWorkgroups) nwg = kMaxResidentWorkgroups;
    // A family: a stage and the stages that add onto its rows on the same workgroups (addend_local), in list order.
    // The phases are cut family by family; a family costs the sum of its members.
    std::vector<int> root((size_t)nstages);
    std::vector<std::vector<int>> family((size_t)nstages);
    for (int s = 0; s < nstages; ++s) {
        root[(size_t)s] = table[(size_t)s].addend_local ? root[(size_t)table[(size_t)s].dep2] : s;
        family[(size_t)root[(size_t)s]].push_back(s);
    }
    std::vector<std::vector<int>> by_phase((size_t)nphases);
    for (int s = 0; s < nstages; ++s)
        if (root[(size_t)s] == s) by_phase[table[s].phase].push_back(s);
    auto family_units = [&](int head) {
        long long u = 0;
        for (int s : family[(size_t)head]) u += table[(size_t)s].units;
        return u;
    };
    // slices per phase and workgroup, in the order in which the workgroup works them off
    std::vector<std::vector<std::vector<nq::RunSegment>>> slice((size_t)nphases);
    for (int ph = 0; ph < nphases; ++ph) {
        slice[ph].resize((size_t)nwg);
        const std::vector<int>& ids = by_phase[ph];
        std::vector<long long> prefix(ids.size() + 1, 0);
        for (size_t k = 0; k < ids.size(); ++k)
            prefix[k + 1] = prefix[k] + (long long)table[ids[k]].rows * family_units(ids[k]);
        const long long total = prefix.back();
        if (ids.size() * 2 <= (size_t)nwg) {
            // Few stages, many workgroups: give every stage whole workgroups, so that no workgroup stages
            // two input vectors in one phase.  A slice costs units * rows + fixed: staging the input vector takes
            // about as long as the arithmetic of `overhead_rows` rows of the same width (a dozen at batch 1; every
            // workgroup stages all batch rows while a row of signs costs the same for 16 columns as for one, so
            // 48 at batch 8 and 64 at batch 16, from phase timelines of Llama-2-7B layers), and every further pass
            // of an input too long to be staged at once costs the latency of one more staging round trip
            // (2 us, 700 row units there).  The workgroup counts n_s minimise the slowest slice,
            // max_s (units_s * rows_s / n_s + fixed_s).
            const double overhead_rows = batch >= 16 ? 64.0 : wide ? 48.0 : 12.0;
            const double pass_cost = wide ? 700.0 : 0.0;
            const int chunk_cap = std::max(1, nq::stream_chunk_cap(dtype, batch, max_units, alt));
            std::vector<double> fixed(ids.size(), 0.0), width(ids.size(), 0.0);
            for (size_t k = 0; k < ids.size(); ++k)
                for (int s : family[(size_t)ids[k]]) {
                    const int u = table[(size_t)s].units;
                    fixed[k] += u * overhead_rows + ((u + chunk_cap - 1) / chunk_cap - 1) * pass_cost;
                    width[k] += u;
                }
            std::vector<int> share(ids.size(), 1);
            auto needed = [&](double t) {       // workgroups needed for every slice to cost at most t
                long long sum = 0;
                for (size_t k = 0; k < ids.size(); ++k) {
                    const double u = width[k], r = table[ids[k]].rows;
                    const double room = t - fixed[k];
                    if (room <= 0) return (long long)nwg + 1;
                    long long n = (long long)((u * r + room - 1e-9) / room);
                    if (n < 1) n = 1;
                    if (n > table[ids[k]].rows) n = table[ids[k]].rows;
                    sum += n;
                }
                return sum;
            };
            double lo = 0, hi = 0;
            for (size_t k = 0; k < ids.size(); ++k) {
                const double t1 = width[k] * table[ids[k]].rows + fixed[k];
                if (t1 > hi) hi = t1;
            }
            for (int iter = 0; iter < 60; ++iter) {
                const double mid = 0.5 * (lo + hi);
                if (needed(mid) <= nwg) hi = mid; else lo = mid;
            }
            int used = 0;
            for (size_t k = 0; k < ids.size(); ++k) {
                const double u = width[k], r = table[ids[k]].rows;
                const double room = hi - fixed[k];
                long long n = room > 0 ? (long long)((u * r + room - 1e-9) / room) : 1;
                if (n < 1) n = 1;
                if (n > table[ids[k]].rows) n = table[ids[k]].rows;
                share[k] = (int)n;
                used += share[k];
            }
            // left-over workgroups go where a slice is slowest
            while (used < nwg) {
                size_t best = ids.size();
                double worst = -1;
                for (size_t k = 0; k < ids.size(); ++k) {
                    if (share[k] >= table[ids[k]].rows) continue;
                    const double t = width[k] * ((double)table[ids[k]].rows / share[k]) + fixed[k];
                    if (t > worst) { worst = t; best = k; }
                }
                if (best == ids.size()) break;
                ++share[best];
                ++used;
            }
            int w = 0;
            for (size_t k = 0; k < ids.size(); ++k) {
                const int rows = table[ids[k]].rows;
                // tile order: cut between the row groups of a wave-load, so that each is one contiguous KiB
                const bool tiled = table[ids[k]].tiled != 0;
                const int ntile = (rows + granule - 1) / granule;
                for (int j = 0; j < share[k]; ++j, ++w) {
                    int rb = (int)((long long)rows * j / share[k]);
                    int re = (int)((long long)rows * (j + 1) / share[k]);
                    if (tiled) {
                        rb = (int)std::min<long long>(rows, (long long)granule * ((long long)ntile * j / share[k]));
                        re = (int)std::min<long long>(rows, (long long)granule * ((long long)ntile * (j + 1) / share[k]));
                    }
                    if (re > rb)
                        for (int s : family[(size_t)ids[k]]) {
                            slice[ph][(size_t)w].push_back(nq::RunSegment{s, rb, re, 0});
                            table[(size_t)s].seg_count += 1;
                        }
                }
            }
            continue;
        }
        // Many stages: every workgroup gets the same COST, cut wherever that falls.  A slice costs its arithmetic
        // (rows x units) plus a fixed part for taking up a new stage: the dependency check, the staging of the input
        // vector (a round trip to memory behind the running stream), the drain of the fetch pipeline and the
        // epilogue, measured at 5.6 us per slice in a 26-layer list at batch 1, where a workgroup streams about
        // 25 KB per us, i.e. 140 KB = 8800 units of arithmetic; equal arithmetic alone left the workgroups with
        // many slices 20 % behind those with few.  The cost T per workgroup is the smallest for which a greedy
        // fill (never starting a slice that cannot hold a quarter of the fixed part in arithmetic) needs at most
        // the resident workgroups.
        {
            // (the variant whose wavefronts own row pairs starts every slice without fetches in flight, so a slice
            // costs it more to start: 16000, and 10000 at batch 1, the best of sweeps on the Llama-2-7B stack)
            const long long fixed_one = own ? (batch == 1 ? 10000 : 16000) : wide ? 2200 : batch == 1 ? 8800 : batch == 2 ? 6600 : 4400;
            auto gran = [&](size_t k) { return table[ids[k]].tiled ? granule : 1; };
            // Batch 8 and 16: an input too long to be staged at once is staged again, chunk by chunk, for every 256 rows
            // of a slice (three barriers and a round trip to memory per chunk): charged as 10 more units per chunk and
            // row, from per-workgroup time accounts of the Llama-2-7B stack (down projection, 86 units in 3 chunks
            // at batch 16: without the charge its workgroups end 20 % behind the others).
            const long long chunk_cap_long = std::max(1, nq::stream_chunk_cap(dtype, batch, max_units, alt));
            auto restage = [&](long long units) -> long long {
                const long long chunks = (units + chunk_cap_long - 1) / chunk_cap_long;
                return wide && chunks > 1 ? 10 * chunks : 0;
            };
            // fills workgroups with budget T; returns how many it needs (emits the slices when `emit`)
            auto fill = [&](long long T, bool emit) -> long long {
                long long w = 0, budget = T;
                size_t k = 0;
                int row = 0;
                while (k < ids.size()) {
                    const nq::RunStage& stg = table[ids[k]];
                    const std::vector<int>& fam = family[(size_t)ids[k]];
                    long long u = 0;
                    for (int s : fam) u += table[(size_t)s].units + restage(table[(size_t)s].units);
                    const long long fixed = fixed_one * (long long)fam.size();
                    const int left = stg.rows - row;
                    const int g = gran(k);
                    const long long least = fixed + u * std::min<long long>(left, std::max<long long>(g, fixed / (4 * u)));
                    if (budget < least) {
                        if (budget == T) return (long long)nwg + 1;     // T cannot hold even the smallest slice
                        ++w;
                        budget = T;
                        continue;
                    }
                    long long fit = (budget - fixed) / u;
                    if (fit < left) fit = fit / g * g;                   // cut between the row groups of a wave-load
                    const int take = (int)std::min<long long>(left, fit);
                    if (emit && w < nwg)
                        for (int s : fam) {
                            slice[ph][(size_t)w].push_back(nq::RunSegment{s, row, row + take, 0});
                            table[(size_t)s].seg_count += 1;
                        }
                    budget -= fixed + u * take;
                    row += take;
                    if (row >= stg.rows) { ++k; row = 0; }
                }
                return w + 1;
            };
            long long lo = total / nwg, hi = 2 * total + (long long)nstages * fixed_one + 1;   // restage() adds at most 10 to chunk_cap + 1 units
            while (lo < hi) {
                const long long mid = lo + (hi - lo) / 2;
                if (fill(mid, false) <= nwg) hi = mid; else lo = mid + 1;
            }
            if (fill(lo, true) > nwg) return NQ_ERR_SHAPE;               // cannot happen: hi always fits
        }
    }
    // Slice records: record w is the first slice of workgroup w (phase by phase, in the order of `slice`), the others
    // follow behind the nwg first records, contiguous per workgroup.  Each record carries a copy of its stage.
    for (auto& st : table) {
        st.dep_segs = st.dep >= 0 ? table[(size_t)st.dep].seg_count : 0;
        st.dep2_segs = st.dep2 >= 0 ? table[(size_t)st.dep2].seg_count : 0;
    }
    std::vector<nq::RunSlice> records((size_t)nwg);
    for (int w = 0; w < nwg; ++w) {
        nq::RunSlice first = {};
        first.seg = nq::RunSegment{-1, 0, 0, 0};
        first.more_begin = first.more_end = (int)records.size();
        bool have_first = false;
        for (int ph = 0; ph < nphases; ++ph)
            for (const auto& sg : slice[ph][w]) {
                nq::RunSlice r = {};
                r.seg = sg;
                r.st = table[(size_t)sg.stage];
                if (!have_first) {
                    r.more_begin = first.more_begin;
                    first = r;
                    have_first = true;
                } else {
                    records.push_back(r);
                }
            }
        first.more_end = (int)records.size();
        records[(size_t)w] = first;
    }

    const size_t off_slices = 256 + runlist_counter_bytes(nlinears);
    if (off_slices + records.size() * sizeof(nq::RunSlice) > workspace_bytes) return NQ_ERR_WORKSPACE;

    hipStream_t hs = (hipStream_t)stream;
    char* base = (char*)workspace;
    hipError_t e = hipMemsetAsync(base, 0, off_slices, hs);
    if (e != hipSuccess) return hip_status(e);
    e = hipMemcpyAsync(base + off_slices, records.data(), records.size() * sizeof(nq::RunSlice), hipMemcpyHostToDevice, hs);
    if (e != hipSuccess) return hip_status(e);
    plan_out->nlinears = nlinears;
    plan_out->nstages = nstages;
    plan_out->nphases = nphases;
    plan_out->workgroups = nwg;
    plan_out->max_units = max_units;
    plan_out->batch = batch;
    plan_out->dtype = dtype;
    plan_out->index_words = (int)records.size();
    plan_out->bound = 0;
    plan_out->spin_limit = 0;
    for (int i = 0; i < nlinears; ++i) plan_out->bound |= (linears[i].x ? 0 : 1) | (linears[i].y ? 0 : 2);
    if (linears[0].tiled) plan_out->bound |= 4;
    if (alt) plan_out->bound |= 16;
    if (own) plan_out->bound |= 32;
    return hip_status(hipStreamSynchronize(hs));   // the tables are host memory: finish before they die
}

int nq_runlist_run(const void* workspace, const nq_runlist_plan* plan, void* stream) {
    return nq_runlist_run_bound(workspace, plan, nullptr, nullptr, stream);
}

int nq_runlist_run_bound(const void* workspace, const nq_runlist_plan* plan, const void* x, void* y, void* stream) {
    if (!workspace || !plan) return NQ_ERR_NULL;
    if (((plan->bound & 1) && !x) || ((plan->bound & 2) && !y)) return NQ_ERR_NULL;
    if (((uintptr_t)x) & 15u) return NQ_ERR_ALIGN;
    if (plan->dtype != NQ_F16 && plan->dtype != NQ_BF16) return NQ_ERR_DTYPE;
    if (plan->nlinears <= 0 || plan->nstages != 2 * plan->nlinears || plan->workgroups <= 0 || plan->max_units <= 0 ||
        plan->nphases <= 0 || plan->index_words < plan->workgroups)
        return NQ_ERR_SHAPE;
    const int batch = plan->batch;
    if (batch != 1 && batch != 2 && batch != 4 && batch != 8 && batch != 16) return NQ_ERR_SHAPE;
    char* base = (char*)workspace;
    const size_t off_slices = 256 + runlist_counter_bytes(plan->nlinears);
    return hip_status(nq::gemv_stream(plan->dtype, batch, plan->nstages, (const nq::RunSlice*)(base + off_slices),
                                      (unsigned long long*)(base + 256),
                                      (unsigned*)base, plan->workgroups, plan->max_units, (hipStream_t)stream, x, y,
                                      (plan->bound & 4) != 0, (plan->bound & 8) != 0,
                                      plan->spin_limit > 0 ? (unsigned)plan->spin_limit : 0u, (plan->bound & 16) != 0,
                                      (plan->bound & 32) != 0));
}

int nq_runlist_capacity(int batch, int dtype, int max_units, int variant) {
    if (dtype != NQ_F16 && dtype != NQ_BF16) return 0;
    if (batch != 1 && batch != 2 && batch != 4 && batch != 8 && batch != 16) return 0;
    if (max_units <= 0 || variant < -1 || variant > 5) return 0;
    return nq::stream_capacity(dtype, batch, max_units, false, variant);
}

int nq_runlist_set_deterministic(nq_runlist_plan* plan, int on) {
    if (!plan) return NQ_ERR_NULL;
    if (plan->dtype != NQ_F16 && plan->dtype != NQ_BF16) return NQ_ERR_DTYPE;
    if (on && !nq::stream_has_deterministic(plan->dtype, plan->batch)) return NQ_ERR_SHAPE;
    plan->bound = on ? (plan->bound | 8) : (plan->bound & ~8);
    return NQ_OK;
}

int nq_runlist_status(const void* workspace, int* status_out, void* stream) {
    if (!workspace || !status_out) return NQ_ERR_NULL;
    unsigned v = 0;
    hipError_t e = hipMemcpyAsync(&v, workspace, sizeof(v), hipMemcpyDeviceToHost, (hipStream_t)stream);
    if (e != hipSuccess) return hip_status(e);
    e = hipStreamSynchronize((hipStream_t)stream);
    *status_out = (int)v;
    if (e == hipSuccess && v != 0) {                 // read and clear: the next launch starts with a clean word
        e = hipMemsetAsync(const_cast<void*>(workspace), 0, sizeof(v), (hipStream_t)stream);
        if (e == hipSuccess) e = hipStreamSynchronize((hipStream_t)stream);
    }
    return hip_status(e);
}

size_t nq_gemm_scratch_bytes(int tokens, int k, int rows) { return nq::gemm_scratch_bytes(tokens, k, rows); }

int nq_gemm_onebit(const void* x, const uint32_t* tiles, const void* s_in, const void* s_out, void* y,
                   void* scratch, size_t scratch_bytes, int tokens, int k, int rows, int dtype, void* stream) {
    return nq_gemm_onebit_bias(x, tiles, s_in, s_out, nullptr, y, scratch, scratch_bytes, tokens, k, rows, dtype, stream);
}

int nq_gemm_onebit_bias(const void* x, const uint32_t* tiles, const void* s_in, const void* s_out, const void* bias,
                        void* y, void* scratch, size_t scratch_bytes, int tokens, int k, int rows, int dtype,
                        void* stream) {
    if (dtype != NQ_F16 && dtype != NQ_BF16) return NQ_ERR_DTYPE;
    if (tokens < 0 || k < 0 || rows < 0) return NQ_ERR_SHAPE;
    if (k % 256 != 0 || rows % 32 != 0) return NQ_ERR_PROB_SHAPE;
    if (tokens == 0 || rows == 0 || k == 0) return NQ_OK;
    if (!x || !tiles || !y) return NQ_ERR_NULL;
    if (((uintptr_t)x | (uintptr_t)tiles | (uintptr_t)y | (uintptr_t)s_in | (uintptr_t)scratch | (uintptr_t)bias) & 15u)
        return NQ_ERR_ALIGN;
    const size_t need = nq::gemm_scratch_bytes(tokens, k, rows);
    if (need > 0 && (!scratch || scratch_bytes < need)) return NQ_ERR_WORKSPACE;
    return hip_status(nq::gemm_onebit(dtype, x, tiles, s_in, s_out, y, (float*)scratch, tokens, k, rows,
                                      (hipStream_t)stream, bias));
}

int nq_gemm_nanoquant(const void* x, const uint32_t* vt_tiles, const uint32_t* u_tiles, const void* s_in,
                      const void* s_mid, const void* s_out, void* h, void* y, void* scratch,
                      size_t scratch_bytes, int tokens, int n, int r, int m, int dtype, void* stream) {
    return nq_gemm_nanoquant_bias(x, vt_tiles, u_tiles, s_in, s_mid, s_out, nullptr, h, y, scratch, scratch_bytes, tokens, n, r,
                                  m, dtype, stream);
}

int nq_gemm_nanoquant_bias(const void* x, const uint32_t* vt_tiles, const uint32_t* u_tiles, const void* s_in,
                           const void* s_mid, const void* s_out, const void* bias, void* h, void* y, void* scratch,
                           size_t scratch_bytes, int tokens, int n, int r, int m, int dtype, void* stream) {
    if (!h) return (tokens == 0 || m == 0) ? NQ_OK : NQ_ERR_NULL;
    int st = nq_gemm_onebit(x, vt_tiles, s_in, s_mid, h, scratch, scratch_bytes, tokens, n, r, dtype, stream);
    if (st != NQ_OK) return st;
    return nq_gemm_onebit_bias(h, u_tiles, nullptr, s_out, bias, y, scratch, scratch_bytes, tokens, r, m, dtype, stream);
}

int nq_gemm_group_max(void) { return nq::gemm_group_max(); }

int nq_gemm_nanoquant_group(const nq_gemm_term* terms, int count, int tokens, int dtype, void* scratch,
                            size_t scratch_bytes, void* stream) {
    return nq_gemm_nanoquant_group_ws(terms, count, tokens, dtype, scratch, scratch_bytes, nullptr, 0, NQ_PANEL_NEVER, stream);
}

// Polls after which a wait of a panel launch gives up (0: the kernel's default).  Process-wide; meant for exercising
// a caller's handling of an expired wait from the host.
static std::atomic<unsigned> g_panel_spin_limit{0};
int nq_gemm_panel_set_spin_limit(unsigned polls) {
    g_panel_spin_limit.store(polls);
    return NQ_OK;
}

size_t nq_gemm_panel_workspace_bytes(void) { return nq::panel_workspace_bytes(); }

int nq_gemm_panel_status(const void* panel_ws, int* status_out, void* stream) {
    if (!panel_ws || !status_out) return NQ_ERR_NULL;
    unsigned v = 0;
    const char* word = (const char*)panel_ws + 64;
    hipError_t e = hipMemcpyAsync(&v, word, sizeof(v), hipMemcpyDeviceToHost, (hipStream_t)stream);
    if (e != hipSuccess) return hip_status(e);
    e = hipStreamSynchronize((hipStream_t)stream);
    *status_out = (int)v;
    if (e == hipSuccess && v != 0) {                 // read and clear
        e = hipMemsetAsync(const_cast<char*>(word), 0, sizeof(v), (hipStream_t)stream);
        if (e == hipSuccess) e = hipStreamSynchronize((hipStream_t)stream);
    }
    return hip_status(e);
}

int nq_gemm_nanoquant_group_ws(const nq_gemm_term* terms, int count, int tokens, int dtype, void* scratch,
                               size_t scratch_bytes, void* panel_ws, size_t panel_ws_bytes, int panel_mode, void* stream) {
    if (dtype != NQ_F16 && dtype != NQ_BF16) return NQ_ERR_DTYPE;
    if (count < 0 || tokens < 0) return NQ_ERR_SHAPE;
    if (panel_mode != NQ_PANEL_AUTO && panel_mode != NQ_PANEL_ALWAYS && panel_mode != NQ_PANEL_NEVER) return NQ_ERR_SHAPE;
    if (count == 0 || tokens == 0) return NQ_OK;
    if (!terms) return NQ_ERR_NULL;
    if (count > nq::gemm_group_max()) return NQ_ERR_SHAPE;
    bool grouped = true;
    for (int i = 0; i < count; ++i) {
        const nq_gemm_term& t = terms[i];
        if (t.n <= 0 || t.r <= 0 || t.m <= 0) return NQ_ERR_SHAPE;
        if (t.n % 256 != 0 || t.r % 256 != 0 || t.m % 32 != 0) return NQ_ERR_PROB_SHAPE;
        if (!t.x || !t.vt_tiles || !t.u_tiles || !t.h || !t.y) return NQ_ERR_NULL;
        if (((uintptr_t)t.x | (uintptr_t)t.vt_tiles | (uintptr_t)t.u_tiles | (uintptr_t)t.h | (uintptr_t)t.y |
             (uintptr_t)t.s_in | (uintptr_t)t.s_mid | (uintptr_t)t.s_out | (uintptr_t)t.bias) & 15u)
            return NQ_ERR_ALIGN;
        if ((t.s_in == nullptr) != (terms[0].s_in == nullptr)) grouped = false;   // one kernel variant per launch
        for (int j = 0; j < i; ++j)
            if (terms[j].h == t.h || terms[j].y == t.y) return NQ_ERR_SHAPE;      // results would overwrite each other
    }
    if (!grouped) {                              // mixed kernel variants: one linear after the other
        for (int i = 0; i < count; ++i) {
            const nq_gemm_term& t = terms[i];
            int st = nq_gemm_nanoquant_bias(t.x, t.vt_tiles, t.u_tiles, t.s_in, t.s_mid, t.s_out, t.bias, t.h, t.y, scratch,
                                            scratch_bytes, tokens, t.n, t.r, t.m, dtype, stream);
            if (st != NQ_OK) return st;
        }
        return NQ_OK;
    }
    constexpr int kMax = 16;                     // >= nq::gemm_group_max(), checked above
    static_assert(kMax >= 16, "group arrays");
    const void* x[kMax]; const uint32_t* w[kMax]; const void* si[kMax]; const void* so[kMax]; const void* bs[kMax]; void* out[kMax];
    int K[kMax], R[kMax];
    if (count > kMax) return NQ_ERR_SHAPE;
    const bool have_ws = panel_ws && panel_mode != NQ_PANEL_NEVER;
    if (have_ws) {
        if (((uintptr_t)panel_ws) & 255u) return NQ_ERR_ALIGN;
        const size_t need = nq::panel_workspace_bytes();
        if (need == 0 || panel_ws_bytes < need) return NQ_ERR_WORKSPACE;
    }
    // one stage: the panel launch where a workspace was given and the shapes make it the faster one
    auto stage = [&]() -> hipError_t {
        if (have_ws && (panel_mode == NQ_PANEL_ALWAYS || nq::panel_applies(count, tokens, K, R)))
            return nq::gemm_panel_group(dtype, count, x, w, si, so, bs, out, tokens, K, R, panel_ws, g_panel_spin_limit.load(),
                                        (hipStream_t)stream);
        return nq::gemm_onebit_group(dtype, count, x, w, si, so, bs, out, tokens, K, R, (hipStream_t)stream);
    };
    for (int i = 0; i < count; ++i) {
        const nq_gemm_term& t = terms[i];
        x[i] = t.x; w[i] = t.vt_tiles; si[i] = t.s_in; so[i] = t.s_mid; bs[i] = nullptr; out[i] = t.h; K[i] = t.n; R[i] = t.r;
    }
    hipError_t e = stage();
    if (e != hipSuccess) return hip_status(e);
    for (int i = 0; i < count; ++i) {
        const nq_gemm_term& t = terms[i];
        x[i] = t.h; w[i] = t.u_tiles; si[i] = nullptr; so[i] = t.s_out; bs[i] = t.bias; out[i] = t.y; K[i] = t.r; R[i] = t.m;
    }
    return hip_status(stage());
}

size_t nq_tiled_words(int rows, int words) {
    if (rows <= 0 || words <= 0) return 0;
    return nq::tiled_word_count(rows, words);
}

int nq_tile_words(const uint32_t* src, uint32_t* dst, int rows, int words, int inverse, void* stream) {
    if (rows < 0 || words < 0) return NQ_ERR_SHAPE;
    if (rows == 0 || words == 0) return NQ_OK;
    if (!src || !dst) return NQ_ERR_NULL;
    if (src == dst) return NQ_ERR_SHAPE;             // a permutation across rows: not in place
    if (((uintptr_t)(inverse ? src : dst)) & 15u) return NQ_ERR_ALIGN;
    return hip_status(nq::tile_words(src, dst, rows, words, inverse ? 1 : 0, (hipStream_t)stream));
}

int nq_repack_words(const uint32_t* src, uint32_t* dst, size_t nwords, int src_order, int dst_order, void* stream) {
    if ((src_order != 0 && src_order != 1) || (dst_order != 0 && dst_order != 1)) return NQ_ERR_ORDER;
    if (nwords == 0) return NQ_OK;
    if (!src || !dst) return NQ_ERR_NULL;
    return hip_status(nq::repack_words(src, dst, nwords, src_order, dst_order, (hipStream_t)stream));
}

int nq_pack_gemm_tiles(const uint32_t* words, uint32_t* tiles, int rows, int words_per_row, int rows_padded,
                       int k_padded, int src_order, void* stream) {
    if (src_order != 0 && src_order != 1) return NQ_ERR_ORDER;
    if (rows < 0 || words_per_row < 0 || rows_padded < rows || (long long)k_padded < 32ll * words_per_row) return NQ_ERR_SHAPE;
    if (rows_padded % 32 != 0 || k_padded % 256 != 0) return NQ_ERR_PROB_SHAPE;
    if (rows_padded == 0 || k_padded == 0) return NQ_OK;
    if (!tiles || (!words && rows > 0 && words_per_row > 0)) return NQ_ERR_NULL;
    if (words == tiles) return NQ_ERR_SHAPE;         // a permutation across words: not in place
    return hip_status(nq::words_to_tiles(words, tiles, rows, words_per_row, rows_padded, k_padded, src_order,
                                         (hipStream_t)stream));
}

int nq_stream_copy(void* dst, const void* src, size_t bytes, void* stream) {
    if (bytes % 16 != 0) return NQ_ERR_SHAPE;
    if (bytes == 0) return NQ_OK;
    if (!src || !dst) return NQ_ERR_NULL;
    return hip_status(nq::stream_copy(dst, src, bytes, (hipStream_t)stream));
}

}  // extern "C"
