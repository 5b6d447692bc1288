/* C ABI of libnq_gfx950.so: the binary low-rank linear layer on AMD gfx950 (MI355X).
 *
 * Every entry point takes raw device pointers, sizes and a HIP stream, enqueues its kernels on that
 * stream and returns without synchronising.  Nothing here allocates or frees device memory and no
 * pointer is kept after return; scratch buffers are passed in by the caller.  Return value: NQ_OK or
 * a negative nq_status; nq_status_string() gives the message (the messages of argument errors are
 * the ones the reference's host wrappers raise).
 *
 * Reference paths are relative to the reference checkout; "kernel/" = src/nanoquant/kernel/.
 * Operand naming follows the mathematics, not the reference's swapped argument names:
 *   vt_bits [r, ceil(n/32)]  first-stage factor  (reference op argument `Ubits`, module attr V_int8)
 *   u_bits  [m, ceil(r/32)]  second-stage factor (reference op argument `Vbits`, module attr U_int8)
 * Packed words use the row-major "half2" order of kernel/utils.py:99-104: element k of a 32-group
 * sits at bit 15 - (k>>1) + 16*(k&1); bit 1 encodes -1, bit 0 encodes +1.
 */
#ifndef NQ_GFX950_H
#define NQ_GFX950_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum nq_dtype { NQ_F16 = 0, NQ_BF16 = 1 } nq_dtype;

typedef enum nq_status {
    NQ_OK = 0,
    NQ_ERR_DTYPE = -1,        /* "Support only Half or BFloat16" (kernel/cuda/gemv_kernel.cu:318) */
    NQ_ERR_NULL = -2,         /* a required pointer is NULL */
    NQ_ERR_SHAPE = -3,        /* a size is negative or inconsistent */
    NQ_ERR_K_MISMATCH = -4,   /* "k dimension mismatch" (kernel/cuda/gemm.cpp:48) */
    NQ_ERR_PROB_SHAPE = -5,   /* "Problem shape incompatible" (kernel/cuda/gemm.cpp:93) */
    NQ_ERR_WORKSPACE = -6,    /* "workspace too small" (kernel/cuda/gemm.cpp:52) */
    NQ_ERR_ORDER = -7,        /* unknown word order id */
    NQ_ERR_ALIGN = -8,        /* a prefill operand is not 16-byte aligned */
    NQ_ERR_SCRATCH_LIMIT = -9, /* nq_gemv_forward_noalloc: batch * r above NQ_NOALLOC_MAX_H_FLOATS */
    NQ_ERR_HIP = -100         /* a HIP call failed; see nq_last_hip_error() */
} nq_status;

typedef enum nq_word_order { NQ_ORDER_LSB_FIRST = 0, NQ_ORDER_HALF2 = 1 } nq_word_order;

typedef enum nq_device_attr { NQ_ATTR_CU_COUNT = 0, NQ_ATTR_LDS_BYTES = 1, NQ_ATTR_WAVE_SIZE = 2 } nq_device_attr;

const char* nq_status_string(int status);
int nq_last_hip_error(void);          /* hipError_t of the most recent NQ_ERR_HIP on this thread */
int nq_abi_version(void);
int nq_device_query(int attr, int* value);   /* current device */

/* Decode path, one term:  y = s_out * (U (s_mid * (Vt (s_in * x)))).
 * Replaces nanoquant_dyn_forward (kernel/cuda/gemv_kernel.cu:308-429; schema kernel/pybind.cpp:86-90).
 *   x [batch, n], s_in [n], s_mid [r] or NULL, s_out [m], y [batch, m]: all of `dtype`, contiguous.
 *   h_scratch: fp32 [batch, r] owned by the caller (the reference allocates `interm` itself, :345).
 * Any batch >= 1 is accepted; every packed word is read once per 16 batch rows. */
int nq_gemv_forward(const void* x, const void* s_in, const uint32_t* vt_bits, const void* s_mid,
                    const uint32_t* u_bits, const void* s_out, float* h_scratch, void* y,
                    int batch, int n, int r, int m, int dtype, void* stream);

/* The same with y += bias (bias [m] of `dtype`, may be NULL), added in the epilogue of the second stage.  The
 * reference's kernel paths drop the bias of a module (modules/linear.py:121-141 returns before :248-257 adds it);
 * this entry point is what a caller uses to keep it. */
int nq_gemv_forward_bias(const void* x, const void* s_in, const uint32_t* vt_bits, const void* s_mid,
                         const uint32_t* u_bits, const void* s_out, const void* bias, float* h_scratch, void* y,
                         int batch, int n, int r, int m, int dtype, void* stream);

/* nq_gemv_forward_bias for callers that cannot allocate device memory or hand over a workspace: code under HIP
 * graph capture, tight serving loops, harnesses that forbid hipMalloc.  No counterpart in the reference (whose
 * wrapper allocates `interm` with torch::empty on every call, kernel/cuda/gemv_kernel.cu:345).  The fp32
 * intermediate h lives in a device array inside the library, NQ_NOALLOC_MAX_H_FLOATS floats (1 MiB) per GPU, held
 * until the process ends: batch * r above that returns NQ_ERR_SCRATCH_LIMIT.  The call allocates and frees nothing.
 * All calls on one GPU share that array: calls that overlap in time on one GPU (two streams, two threads) race on
 * it; h is fully rewritten by every call, nothing needs clearing between calls.  The first call on each device
 * looks up the array's address and should be made outside graph capture. */
#define NQ_NOALLOC_MAX_H_FLOATS (256 * 1024)
int nq_gemv_forward_noalloc(const void* x, const void* s_in, const uint32_t* vt_bits, const void* s_mid,
                            const uint32_t* u_bits, const void* s_out, const void* bias, void* y,
                            int batch, int n, int r, int m, int dtype, void* stream);

/* Decode path, sum of `nterms` terms that share x (the mixture-of-rank layer; no counterpart in the
 * reference's code, defined as the sum of single-term layers).  Arrays hold one pointer / rank per
 * term; s_mid[t] may be NULL.  h_scratch: fp32 [batch, max r]; y_scratch: fp32 [batch, m]. */
int nq_gemv_mixture(const void* x, const void* const* s_in, const uint32_t* const* vt_bits,
                    const void* const* s_mid, const uint32_t* const* u_bits, const void* const* s_out,
                    const int* r, int nterms, float* h_scratch, float* y_scratch, void* y,
                    int batch, int n, int m, int dtype, void* stream);

/* Decode path, run-list form: a whole list of linears (a decoder layer, a decoder stack) in ONE
 * kernel launch.  No counterpart in the reference, which launches two kernels per linear
 * from Python (modules/linear.py:121-130 -> kernel/cuda/gemv_kernel.cu:406-425); it exists because a
 * 1-bit linear is worth well under a microsecond of HBM time and launch boundaries would dominate.
 *
 * nq_linear describes one linear with the operand meaning of nq_gemv_forward; h is its private fp32
 * [batch, r] intermediate.  x_from >= 0 says that x is the y of that earlier entry of the list (the
 * kernel then orders the two); y_from >= 0 says that `addend` is the fp32 y of that earlier entry.
 * With out_f32 the result y is stored as fp32 (used for sums over terms); addend (fp32 [batch, m])
 * is added before the store.  Where the adding entry's own intermediate is ready in time, the builder cuts
 * its second stage into the same rows on the same workgroups as the entry it adds onto, each slice right
 * behind the one that writes its addend, and the two wait for nothing between them.
 *
 * nq_runlist_build writes the stage table into `workspace` (device memory of at least
 * nq_runlist_workspace_bytes(linears, nlinears) bytes, 256-byte aligned) -- it copies from host memory, so it
 * synchronises with the host and must not be captured in a graph.  Stages are grouped into phases by
 * dependency depth and every resident workgroup gets an equal share of every phase, so all linears
 * of a list need distinct h buffers.  `interleave` >= 1 is an ordering hint kept for interface
 * stability; the phase schedule does not need it.
 * nq_runlist_run enqueues the single launch; it allocates nothing and can be graph-captured.  Runs of
 * the same workspace must not overlap in time.  batch must be 1, 2, 4, 8 or 16.
 * Inside the launch a stage waits for the stages it depends on through device-scope counters, which needs every
 * workgroup of the grid resident at once.  The grid is sized to what the device keeps resident when it has the
 * device to itself: a run list must not share the GPU with other kernels (another stream, another process) while
 * it runs.  The waits are bounded: if producers cannot become resident, waiting workgroups give up, set the status
 * word and the grid drains; the outputs of that launch are then invalid.
 * nq_runlist_status copies the status word back (synchronises) and clears it: 0 ok, 1 = a bounded dependency wait
 * expired in some launch since the last call (results invalid; the list itself stays usable). */
typedef struct nq_linear {
    const void* x;          /* NULL: bound at run time (nq_runlist_run_bound) */
    const void* s_in;
    const uint32_t* vt_bits;
    const void* s_mid;      /* may be NULL */
    const uint32_t* u_bits;
    const void* s_out;
    float* h;
    void* y;                /* NULL: bound at run time */
    const float* addend;    /* may be NULL */
    int n, r, m;
    int x_from;             /* -1: x is an external input */
    int y_from;             /* -1: addend (if any) is an external input */
    int out_f32;
    const void* bias;       /* [m] of the list's dtype, added after s_out (before addend); may be NULL */
    int tiled;              /* vt_bits and u_bits are in the tile order of nq_tile_words (16-byte aligned) */
} nq_linear;

/* Launch geometry of a built run list; filled by nq_runlist_build, passed back to nq_runlist_run. */
typedef struct nq_runlist_plan {
    int nlinears, nstages, nphases, workgroups, max_units, batch, dtype, index_words;
    int bound;              /* bit 0: some x was NULL, bit 1: some y was NULL (nq_runlist_run_bound must supply them);
                               bit 2: the linears are in tile order (up to batch 4 all linears of a list must agree);
                               bit 3: reproducible sums (nq_runlist_set_deterministic);
                               bit 4: set by the builder for a short fp16 list at batch 4, which runs on the arithmetic of
                               batch 8 and 16 (16-bit operands; reproducible with or without bit 3);
                               bit 5: set by the builder where the kernel variant whose wavefronts own whole row pairs
                               is the faster one (batch 4, long lists at batch 1 and 2; used for tile order) */
    int spin_limit;         /* polls after which a dependency wait gives up and sets the status word; 0 (as built) =
                               the default of 2^21 polls, about a second.  The caller may lower it, e.g. to exercise
                               its handling of an expired wait: every kernel still runs to its end */
} nq_runlist_plan;

size_t nq_runlist_workspace_bytes(const nq_linear* linears, int nlinears);
int nq_runlist_build(const nq_linear* linears, int nlinears, int batch, int dtype, int interleave,
                     void* workspace, size_t workspace_bytes, nq_runlist_plan* plan_out, void* stream);
int nq_runlist_run(const void* workspace, const nq_runlist_plan* plan, void* stream);
/* The same with the input and output that the list left open: every nq_linear whose x is NULL reads `x`
 * ([batch, n] of the list's dtype, 16-byte aligned; they must agree on n), at most one linear may leave y NULL and it writes `y`.
 * Lets one built list serve a module whose activations live somewhere else on every call (one launch per linear
 * instead of the reference's two, modules/linear.py:121-130).  Linears with a NULL x or y must not be referred to
 * by x_from / y_from. */
int nq_runlist_run_bound(const void* workspace, const nq_runlist_plan* plan, const void* x, void* y, void* stream);
int nq_runlist_status(const void* workspace, int* status_out, void* stream);
/* Workgroups of the run-list kernel that the current device keeps resident at once, for lists of this batch size and
 * type whose longest input has `max_units` 16-byte units per row (plan.max_units).  variant -1: the smallest over all
 * kernel variants a plan can be launched with (row-major or tile order, with or without reproducible sums, wavefronts
 * owning row pairs), which is what nq_runlist_build sizes the grid with; 0..5: one variant (0 where it does not
 * exist).  nq_runlist_run checks the grid against the variant it starts and returns NQ_ERR_HIP
 * (hipErrorLaunchOutOfResources) instead of launching a grid that cannot be resident.  0 on error. */
int nq_runlist_capacity(int batch, int dtype, int max_units, int variant);
/* Reproducible sums for the launches of this plan, on (1) or off (0, as built).  The run-list kernel finishes a row
 * sum with additions from several wavefronts whose order differs from launch to launch, so outputs may differ in
 * the last bit between launches (the reference's reductions are ordered: kernel/cuda/gemv_kernel.cu:148-170,
 * shuffles inside one warp).  With this switch every launch of the plan gives bit-identical outputs.  Batch 1, 2 and
 * 4: partial sums are rounded to a grid on which their additions are exact; the results stay within the same
 * tolerance but lose up to 16 bits below (columns x largest input value); plans with bit 5 of `bound` set in tile
 * order form every row sum in one wavefront and lose nothing (the switch only fixes the order in which the input totals
 * are added).  Batch 8 and 16, and plans with bit 4 of `bound` set: every row sum is formed by one wavefront in a fixed
 * order whether the switch is on or off; it is accepted and selects the same kernel.
 * NQ_ERR_SHAPE for a batch size without a run-list kernel.  Sets bit 3 of plan->bound. */
int nq_runlist_set_deterministic(nq_runlist_plan* plan, int on);

/* Decode path for a group of independent linears: the q/k/v or gate/up projections of a decoder layer in two kernel
 * launches per nq_gemv_group_max() linears (all first stages, then all second stages) instead of the two launches
 * per linear of nq_gemv_forward and of the reference (kernel/cuda/gemv_kernel.cu:406-425), without a built run list:
 * nothing to prepare, any pointers on every call, no requirement on what else the GPU runs.
 *   linears: x_from = y_from = -1, no addend, out_f32 = 0, tiled = 0; h buffers distinct, fp32 [batch, r] each.
 *   Pieces of 1, 2 and 4 batch rows are grouped; pieces of 8 and 16 rows take two launches per linear.
 * one_launch = 1: ONE ordinary launch per group instead of two.  The workgroups of the second stages sit behind those
 * of the first in the same grid, fetch their first sign words, and wait on flags until their linear's h is complete
 * (workgroups start in the order of their ids, so whatever a workgroup waits for is running or done: no resident
 * grid is needed).  On MI355X the signalling through device-coherent memory costs more than the launch boundary it
 * replaces (a Llama-2-7B layer at batch 1 in four groups: 82 us with one launch per group, 48 us with two); the
 * switch is kept for measurement and for callers that are charged per launch.  Its flags live in a device
 * array inside the library (4.5 MiB per GPU, 256 slots dealt round robin, every launch puts its slot back to zero);
 * the first call on each device looks up its address and should be made outside graph capture.  The wait is bounded
 * (2^20 polls): if it expires the launch still ends, its outputs are invalid, and nq_gemv_group_status reports 1.
 * nq_gemv_group_status copies the device's status word back (synchronises `stream`) and clears it. */
int nq_gemv_group_max(void);
int nq_gemv_forward_group(const nq_linear* linears, int count, int batch, int dtype, int one_launch, void* stream);
int nq_gemv_group_status(int* status_out, void* stream);
/* Polls after which the wait of a one_launch group gives up (0 = the default of 2^20).  Process-wide.  Lowering it to 1
 * makes a launch report an expiry at once, which is how a caller's handling of status 1 can be exercised from the
 * host; every kernel still runs to its end. */
int nq_gemv_group_set_spin_limit(unsigned polls);

/* One matmul-free stage: out[b,row] = s_row[row] * sum_c sgn(bits[row,c]) * in[b,c] * s_col[c].
 * Replaces nanoquant_stage1_dyn_kernel / nanoquant_stage2_dyn_kernel launches
 * (kernel/cuda/gemv_kernel.cu:283-301).  in/out are `dtype`; s_col, s_row may be NULL. */
int nq_gemv_stage(const void* in, const void* s_col, const uint32_t* bits, const void* s_row, void* out,
                  int batch, int cols, int rows, int dtype, void* stream);

/* Prefill path, single matrix:  y[t, j] = s_out[j] * sum_k (x[t, k] * s_in[k]) * sgn(W)[j, k].
 * Replaces marlin_onebit_cuda (kernel/cuda/gemm.cpp:59-98; schema kernel/pybind.cpp:93-98).
 *   x [tokens, k], y [tokens, rows], s_in [k] or NULL, s_out [rows] or NULL: `dtype`, contiguous.
 *   tiles: k*rows/32 words in the 32-row x 256-k tile layout of the package's prefill packer (the
 *   layout is private to packer and kernel, as the reference's Marlin layout is).
 *   Requires k % 256 == 0 and rows % 32 == 0 (else NQ_ERR_PROB_SHAPE, the reference's error class
 *   for shapes its tiles do not cover).  scratch: nq_gemm_scratch_bytes(tokens, k, rows) bytes of
 *   device memory (may be NULL when that is 0).  It holds fp32 partial sums and tile counters when k
 *   is split; it MUST BE ZERO ON ENTRY and is zero again when the enqueued work has finished, so a
 *   caller zeroes it once and reuses it (calls sharing a scratch must not overlap in time). */
size_t nq_gemm_scratch_bytes(int tokens, int k, int rows);
int nq_gemm_onebit(const void* x, const uint32_t* tiles, const void* s_in, const void* s_out, void* y,
                   void* scratch, size_t scratch_bytes, int tokens, int k, int rows, int dtype, void* stream);
/* The same with y[t, j] += bias[j] (bias [rows] of `dtype`, 16-byte aligned, may be NULL). */
int nq_gemm_onebit_bias(const void* x, const uint32_t* tiles, const void* s_in, const void* s_out, const void* bias,
                        void* y, void* scratch, size_t scratch_bytes, int tokens, int k, int rows, int dtype,
                        void* stream);

/* Prefill path, one term: two chained one-bit GEMMs with the intermediate h [tokens, r] (`dtype`,
 * caller-owned) between them.  Replaces marlin_nanoquant_cuda (kernel/cuda/gemm.cpp:112-122; schema
 * kernel/pybind.cpp:99-104).  vt_tiles: first stage [r rows x n], u_tiles: second stage [m rows x r];
 * r is the padded rank (multiple of 256, padded entries carry a zero s_mid).
 * scratch: max of nq_gemm_scratch_bytes(tokens, n, r) and nq_gemm_scratch_bytes(tokens, r, m). */
int nq_gemm_nanoquant(const void* x, const uint32_t* vt_tiles, const uint32_t* u_tiles, const void* s_in,
                      const void* s_mid, const void* s_out, void* h, void* y, void* scratch,
                      size_t scratch_bytes, int tokens, int n, int r, int m, int dtype, void* stream);
/* The same with the bias [m] added in the epilogue of the second GEMM (may be NULL). */
int nq_gemm_nanoquant_bias(const void* x, const uint32_t* vt_tiles, const uint32_t* u_tiles, const void* s_in,
                           const void* s_mid, const void* s_out, const void* bias, void* h, void* y, void* scratch,
                           size_t scratch_bytes, int tokens, int n, int r, int m, int dtype, void* stream);

/* Several terms with the same token count in two launches instead of two per term: the first GEMMs of all
 * terms, then the second ones (the projections of a decoder block that read the same tokens: q/k/v, gate/up, or
 * independent linears of a layer).  Up to 128 tokens a single term cannot fill the device and is bound by launch
 * and load latencies; grouped, the same launches carry several times the work.  Above 160 tokens the group runs
 * on 64-token block tiles whose workgroups walk the whole k of their term (no k-split, no scratch): together the
 * terms fill the device where one term needs a k-split and a finish launch to do so.  Only when some terms have
 * s_in and others do not does the call run the terms one after another (nq_gemm_nanoquant_bias); it then needs
 * their scratch, max over terms of nq_gemm_scratch_bytes for both GEMMs (may be NULL otherwise).
 * count <= nq_gemm_group_max(); h and y of different terms must not coincide.  No counterpart in the reference, which launches each linear by itself
 * (modules/linear.py:131-133). */
typedef struct nq_gemm_term {
    const void* x;               /* [tokens, n] */
    const uint32_t* vt_tiles;    /* first stage, [r rows x n] in the prefill tile layout */
    const uint32_t* u_tiles;     /* second stage, [m rows x r] */
    const void* s_in;            /* [n] or NULL (all terms alike) */
    const void* s_mid;           /* [r] or NULL */
    const void* s_out;           /* [m] or NULL */
    const void* bias;            /* [m] or NULL */
    void* h;                     /* [tokens, r] */
    void* y;                     /* [tokens, m] */
    int n, r, m;                 /* n % 256 == 0, r % 256 == 0, m % 32 == 0 */
} nq_gemm_term;
int nq_gemm_group_max(void);
int nq_gemm_nanoquant_group(const nq_gemm_term* terms, int count, int tokens, int dtype, void* scratch,
                            size_t scratch_bytes, void* stream);

/* The same with a workspace for the panel launches.  From about 100 to 768 tokens a group that gives every
 * workgroup a few k steps of work runs a stage as ONE persistent launch (two workgroups per compute unit) over panels
 * of 64 tokens x 256 rows whose k ranges are shared out evenly over the workgroups (what the reference's stream-k
 * stripes do, kernel/cuda/gemm_kernel.cu:335-400, :594-640): panels cut by a share boundary are finished together by
 * the workgroups that end inside them, which exchange partial fp32 tiles through `panel_ws`.
 *   panel_ws: nq_gemm_panel_workspace_bytes() bytes of device memory, 256-byte aligned, ZERO when first used and
 *   left to these launches from then on (it holds partial tiles, hand-over flags and a count of finished
 *   workgroups from which every launch derives its own flag value, so nothing is cleared between launches or graph
 *   replays).  It must not be `scratch` and launches that share it must not overlap in time.
 *   panel_mode: NQ_PANEL_AUTO picks per stage (other token counts and small groups take the launches of
 *   nq_gemm_nanoquant_group), NQ_PANEL_ALWAYS forces the panel launch for any token count, NQ_PANEL_NEVER (or
 *   panel_ws NULL) never takes it.
 * A panel launch keeps two workgroups per compute unit resident and its workgroups wait for each other's partial
 * tiles: it may share the GPU with other kernels (its waits then last until those free their compute units), but a
 * wait that outlasts its bound (2^20 polls, about a second) invalidates the launch's outputs.
 * The waits of a finishing workgroup are bounded; nq_gemm_panel_status copies the workspace's status word back
 * (synchronises) and clears it: 0 ok, 1 = a wait expired in some launch since the last call (that launch's outputs
 * are invalid; the workspace stays usable). */
enum { NQ_PANEL_AUTO = 0, NQ_PANEL_ALWAYS = 1, NQ_PANEL_NEVER = 2 };
size_t nq_gemm_panel_workspace_bytes(void);
int nq_gemm_nanoquant_group_ws(const nq_gemm_term* terms, int count, int tokens, int dtype, void* scratch,
                               size_t scratch_bytes, void* panel_ws, size_t panel_ws_bytes, int panel_mode, void* stream);
int nq_gemm_panel_status(const void* panel_ws, int* status_out, void* stream);
/* Polls after which a wait of a panel launch gives up (0 = the default of 2^20).  Process-wide; for exercising a
 * caller's handling of status 1 from the host, as nq_gemv_group_set_spin_limit. */
int nq_gemm_panel_set_spin_limit(unsigned polls);

/* Word-order conversion on the device, in place allowed (dst == src): the checkpoint format
 * ("lsb_first", modules/linear.py:298) to the kernel format ("half2", modules/linear.py:171-172)
 * without the dense round trip of utils/load_utils.py:269-293.  order ids: nq_word_order. */
int nq_repack_words(const uint32_t* src, uint32_t* dst, size_t nwords, int src_order, int dst_order, void* stream);

/* Row-major packed words of a factor (either word order) -> the 32-row x 256-k tile layout that the prefill
 * entry points read, on the device and without a dense matrix: the second half of serving a checkpoint
 * (modules/linear.py:288-321 writes `lsb_first` words [rows, ceil(cols/32)]; utils/load_utils.py:269-293 unpacks
 * them to dense +-1 before kernel/utils.py:217-284 packs them again).  words [rows, words_per_row]; tiles receives
 * rows_padded * k_padded / 32 words; rows_padded % 32 == 0, k_padded % 256 == 0, rows_padded >= rows,
 * k_padded >= 32 * words_per_row.  Rows and columns beyond the source are +1 signs (zero bits): the rank padding
 * of the two-stage packer (kernel/utils.py:262-271), to be paired with a zero mid scale.  src != dst. */
int nq_pack_gemm_tiles(const uint32_t* words, uint32_t* tiles, int rows, int words_per_row, int rows_padded,
                       int k_padded, int src_order, void* stream);

/* Tile order of the packed words for run lists (no counterpart in the reference, whose kernels read the row-major
 * words of kernel/utils.py:51-113 directly): 16-byte units indexed [row/32][unit/4][(row/16)&1][unit&3][row&15],
 * rows padded to a multiple of 32 and units (4 words) to a multiple of 4 with zero words.  The 64 units a wavefront
 * fetches for one MFMA operand are then 1 KiB contiguous instead of 16 pieces of 64 bytes, worth 15-25 % of read
 * bandwidth in long run lists.  nq_tiled_words: 32-bit words of the tiled buffer.  nq_tile_words: row-major
 * [rows, words] -> tile order, or back with inverse != 0; src and dst must differ; the tiled side must be 16-byte
 * aligned. */
size_t nq_tiled_words(int rows, int words);
int nq_tile_words(const uint32_t* src, uint32_t* dst, int rows, int words, int inverse, void* stream);

/* Plain device copy kernel of known traffic (bytes read + bytes written); used to calibrate the
 * memory counters of a profiler.  bytes must be a multiple of 16. */
int nq_stream_copy(void* dst, const void* src, size_t bytes, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* NQ_GFX950_H */
