/*
 * f8mi.h -- C ABI of libf8mi.so: the Float8Linear training hot path of
 * pytorch-labs/float8_experimental as hand-written gfx950 (MI355X) kernels.
 *
 * Conventions
 *   - Every pointer named `*_dev`, every tensor pointer and every workspace is
 *     DEVICE memory owned by the caller.  The library never allocates, frees or
 *     synchronises; every call only enqueues kernels on `stream` (a
 *     hipStream_t passed as void*; NULL = the default stream).
 *   - Calls are re-entrant and may come from any host thread (autograd runs the
 *     backward on its own thread).
 *   - Return value: F8MI_OK or a negative F8MI_ERR_* code; f8mi_last_error()
 *     gives the calling thread's last message.
 *   - "scale" always has the reference's meaning: high precision * scale = fp8
 *     range (float8_tensor.py:252-255 of the reference).
 *
 * Paths cited below are relative to the reference checkout
 * (pytorch-labs/float8_experimental).
 */
#ifndef F8MI_H
#define F8MI_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define F8MI_VERSION 110

#define F8MI_OK 0
#define F8MI_ERR_INVALID_ARG (-1) /* null pointer, negative size, unknown enum            */
#define F8MI_ERR_UNSUPPORTED (-2) /* valid request this build does not implement          */
#define F8MI_ERR_HIP (-3)         /* a HIP runtime call failed (launch, event, ...)       */
#define F8MI_ERR_ARCH (-4)        /* the current device is not gfx950                     */

/* element type of a high-precision tensor, and the dtype arithmetic is rounded to */
#define F8MI_BF16 0
#define F8MI_FP16 1
#define F8MI_FP32 2

/* OCP fp8 formats (torch.float8_e4m3fn / torch.float8_e5m2; float8_utils.py:31-32) */
#define F8MI_E4M3FN 0
#define F8MI_E5M2 1

/* kernel ids for the profiling counters */
#define F8MI_K_AMAX 0
#define F8MI_K_CAST 1
#define F8MI_K_GEMM 2
#define F8MI_K_SYNC 3
#define F8MI_K_COUNT 4

int f8mi_version(void);
const char* f8mi_last_error(void);

/* "" for the library as shipped.  A measurement build (compiled with one of the knobs of csrc/f8mi_knobs.h set: another
 * tile walk, cache policy, ...) answers with the knobs' names and values, so that callers and benchmarks can tell
 * and record which build they run.  Every knob leaves results unchanged.  No counterpart in the reference. */
const char* f8mi_build_knobs(void);

/* Fills CU count, LDS bytes per workgroup and the gcn arch name of HIP device `device`.
 * Returns F8MI_ERR_ARCH when it is not a gfx950. */
int f8mi_device_info(int device, int* cu_count, int* lds_bytes, char* arch, int arch_len);

/* Bytes of the small device workspace f8mi_amax_scale needs (per-block partial
 * results; 4 KB).  Its contents between calls do not matter.  One workspace must
 * not be shared by calls that can overlap in time (use one per stream). */
size_t f8mi_workspace_bytes(void);

/*
 * amax = max|x| and the fp8 scale derived from it, in one pass over x.
 * Replaces tensor_to_amax (float8_utils.py:102-112) + amax_to_scale
 * (float8_utils.py:35-57), i.e. tensor_to_scale (float8_utils.py:115-120).
 *   x          rows x cols elements of `in_dtype`, row stride `ld` elements (ld >= cols), or ld = 0: every row is
 *              the same `cols` elements -- a broadcast row, as autograd hands an expanded gradient
 *              (float8_scaling_utils.py:204-216 receives y.sum().backward()'s dY that way); f8mi_cast and
 *              f8mi_cast_dynamic take ld = 0 likewise, and only `cols` elements are read
 *   math_dtype dtype each step of `fmax / clamp(amax, 1e-12)` is rounded to:
 *              `in_dtype` for dynamic scaling (the reference computes the scale
 *              in the tensor's dtype), F8MI_FP32 for delayed-scaling buffers
 *   orig_is_fp16  clamp the scale to 65504 (float8_utils.py:54-55)
 *   amax_dev   out, 1 float (the amax widened to fp32), may be NULL
 *   scale_dev  out, 1 float, may be NULL
 * NaN anywhere in x gives NaN amax and NaN scale, like torch.max.
 */
int f8mi_amax_scale(const void* x, int64_t rows, int64_t cols, int64_t ld, int in_dtype, int fp8_fmt,
                    int math_dtype, int orig_is_fp16, float* amax_dev, float* scale_dev, void* workspace,
                    void* stream);

/* One tensor of a list given to f8mi_amax_scale_multi. */
typedef struct f8mi_tensor_ref {
    const void* data;   /* dense, 16-byte aligned, `numel` elements of the call's in_dtype */
    int64_t numel;
    int64_t first_tile; /* number of tiles of all entries before this one; an entry has
                           numel / f8mi_amax_tile_elems(in_dtype) + 1 tiles */
} f8mi_tensor_ref;

/* Elements of `in_dtype` in one tile (32 KB) of f8mi_amax_scale_multi's numbering. */
int64_t f8mi_amax_tile_elems(int in_dtype);

/*
 * amax and scale of n tensors in one pass: amax_dev[i], scale_dev[i] (either may be NULL) as
 * f8mi_amax_scale gives them for tensor i.  Replaces the torch._foreach_norm(weights, ord=inf)
 * + stack + clamp + divide chain of precompute_float8_dynamic_scale_for_fsdp
 * (fsdp_utils.py:59-66) -- the per-GPU part of it; the all-reduce between ranks is the caller's.
 *   refs_dev     device array of n entries (n <= f8mi_workspace_bytes() / 4)
 *   total_tiles  sum of the entries' tile counts
 * Three launches whatever n is.
 */
int f8mi_amax_scale_multi(const f8mi_tensor_ref* refs_dev, int n, int64_t total_tiles, int in_dtype, int fp8_fmt,
                          int math_dtype, int orig_is_fp16, float* amax_dev, float* scale_dev, void* workspace,
                          void* stream);

/*
 * Saturated cast to fp8: bytes = fp8(clamp(x * scale, -fmax, fmax)), round to
 * nearest even.  Replaces _ToFloat8ConstrFunc.forward (float8_tensor.py:139-191)
 * + to_fp8_saturated (float8_utils.py:123-139), and the fp8 transpose copies
 * that preprocess_addmm makes for the backward GEMMs (float8_ops.py:131-155).
 *   scale_dev      1 float in device memory
 *   product_dtype  dtype `x * scale` is rounded to before clamp + conversion:
 *                  `in_dtype` when the reference's scale is a 0-dim tensor
 *                  (dynamic scaling), F8MI_FP32 when it is the [1]-shaped buffer
 *                  of delayed scaling or x is fp32
 *   out            rows x cols bytes, dense row-major; may be NULL
 *   out_t          cols x rows bytes, dense (the transpose); may be NULL
 *   amax_dev       if not NULL, max|x| of THIS call is stored there (fused
 *                  amax for hp_tensor_to_float8_delayed,
 *                  float8_scaling_utils.py:65-96)
 *   workspace      reserved; may be NULL
 */
int f8mi_cast(const void* x, int64_t rows, int64_t cols, int64_t ld, int in_dtype, const float* scale_dev,
              int product_dtype, int fp8_fmt, uint8_t* out, uint8_t* out_t, float* amax_dev, void* workspace,
              void* stream);

/*
 * C[m][n] = (sum_k A[m][k] * Bt[n][k]) * (1/scale_a) * (1/scale_b) (+ bias[n]),
 * fp32 accumulation on the fp8 matrix cores.  Replaces addmm_float8_unwrapped
 * -> torch._scaled_mm (float8_python_api.py:24-64) as reached from float8_mm
 * (float8_ops.py:158-190).  Both operands are contiguous along k (A row-major,
 * B column-major in the reference's words): forward x*W^T, grad_input dY*W and
 * grad_weight dY^T*x all have this form once the transposed copies exist.
 * Any m, n, k >= 0 is accepted (ragged edges are handled in the kernel).  Up to 16 rows of A (up to 256
 * while streaming Bt once per 128 rows beats a round of 128-row tiles: a narrow Bt) with k % 128 == 0 take a
 * kernel that reads Bt at memory speed (an inference decode step); it sums the products in another order
 * than the tile kernels, so its results agree with theirs within the accumulation tolerance, not bit for bit.
 * Which kernel runs depends on (m, n, k) and alignment only.
 *   a_fmt/b_fmt   F8MI_E4M3FN / F8MI_E5M2 per operand
 *   lda/ldb       row strides in bytes (>= k)
 *   scale_a_dev, scale_b_dev   the operands' forward scales (1 float each)
 *   c_dtype       F8MI_BF16 / F8MI_FP16 / F8MI_FP32, ldc in elements
 *   bias_dev      n elements of c_dtype, or NULL
 */
int f8mi_gemm_nt(const void* a, int a_fmt, int64_t lda, const void* bt, int b_fmt, int64_t ldb, int64_t m,
                 int64_t n, int64_t k, const float* scale_a_dev, const float* scale_b_dev, void* c, int c_dtype,
                 int64_t ldc, const void* bias_dev, void* stream);

/* ---- k-blocked operands: the layout the fused Float8Linear path keeps its fp8 copies in ----
 * A GEMM operand with R rows and contraction length kc (a multiple of 64) is stored as
 * [kc/64][R][64]: byte (r, k) sits at ((k/64)*R + r)*64 + k%64.  The 64-deep slab of 256 rows
 * that a workgroup consumes per step is then 16 KB of consecutive memory instead of 256 pieces
 * of 64 bytes, which the load unit and the L2 move measurably faster (whole cache lines, even
 * channel spread).  The reference keeps fp8 data row-major only (float8_tensor.py:250-262,
 * float8_ops.py:150-153); these two entry points have no counterpart there and never change
 * values, only where bytes are put.
 */
#define F8MI_LAYOUT_ROWMAJOR 0
#define F8MI_LAYOUT_KBLOCK64 1
/* The same layout for ANY contraction length: the contraction is extended with zero bytes to f8mi_padded_k(kc), the
 * next multiple of 128, and stored [f8mi_padded_k(kc)/64][R][64].  Zeros add nothing to a product, so a GEMM over the
 * padded length gives the product of the unpadded operands -- what the reference's pad_tensor_for_matmul does to the
 * inner dimension of a ragged layer before torch._scaled_mm (float8_utils.py:206-247, float8_ops.py:139-149), here
 * done by the cast kernel as it writes the copy.  Output only: the GEMM entry points take such an operand as an
 * ordinary k-blocked one of contraction length f8mi_padded_k(kc). */
#define F8MI_LAYOUT_KBLOCK64_PAD128 2

/* Contraction length of a F8MI_LAYOUT_KBLOCK64_PAD128 operand: k rounded up to a multiple of 128 (pure arithmetic). */
int64_t f8mi_padded_k(int64_t k);

/* f8mi_cast with a layout per output.  out_layout = KBLOCK64 stores `out` as [cols/64][rows][64]
 * (needs cols % 64 == 0), out_t_layout = KBLOCK64 stores the transpose as [rows/64][cols][64]
 * (needs rows % 64 == 0).  KBLOCK64_PAD128 takes any shape: `out` is [f8mi_padded_k(cols)/64][rows][64] and `out_t`
 * [f8mi_padded_k(rows)/64][cols][64] bytes, every byte of which is written (zeros past the tensor's edge, also
 * when the scale is NaN).  The input's rows need no alignment beyond the element's own: eight elements are one
 * 16-byte load at any row pitch.  Everything else as f8mi_cast. */
int f8mi_cast_layout(const void* x, int64_t rows, int64_t cols, int64_t ld, int in_dtype, const float* scale_dev,
                     int product_dtype, int fp8_fmt, uint8_t* out, int out_layout, uint8_t* out_t, int out_t_layout,
                     float* amax_dev, void* stream);

/* Delayed scaling in one call: f8mi_cast_layout with the module's existing scale (the product x * scale in fp32, as
 * with the [1]-shaped scale buffer), and *amax_dev = max|x| of this call -- hp_tensor_to_float8_delayed
 * (float8_scaling_utils.py:65-96: amax_buffer.fill_(tensor_to_amax(x)), then the cast with the stale scale).
 * Same bytes and the same amax as f8mi_cast_layout with amax_dev; what differs is how the amax leaves the cast kernel:
 * there every workgroup compares with *amax_dev at its end (and holds its LDS and wave slots for that round trip:
 * 6 - 20 us per tensor of 128 MB - 1.8 GB), here every wave folds its maximum into one of 1024 words of `workspace`
 * with an atomic that returns nothing, and a one-workgroup launch reduces the words (4 us).
 *   workspace   f8mi_delayed_workspace_bytes() of device memory, 4-byte aligned, ALL ZERO before the first call that
 *               uses it; every call leaves it all zero again when its work completes.  Not to be shared by calls that
 *               can overlap in time (one per stream), and not the workspace of f8mi_amax_scale, whose contents are
 *               arbitrary. */
size_t f8mi_delayed_workspace_bytes(void);
int f8mi_cast_delayed(const void* x, int64_t rows, int64_t cols, int64_t ld, int in_dtype, const float* scale_dev, int fp8_fmt,
                      uint8_t* out, int out_layout, uint8_t* out_t, int out_t_layout, float* amax_dev, void* workspace,
                      void* stream);

/* Dynamic scaling in one call: scale = f8mi_amax_scale(x) in x's own dtype, then f8mi_cast_layout(x, scale) with the
 * product in x's dtype -- hp_tensor_to_float8_dynamic (float8_scaling_utils.py:33-62: tensor_to_scale, then
 * hp_tensor_and_scale_to_float8 with the 0-dim scale).  *scale_dev receives the scale.  A tensor of at most
 * 32 K elements goes through one launch of one workgroup (a few rows of activations: the launches cost more
 * than the work), anything larger through the two kernels above; the results are the same bits either way.
 * `workspace` as for f8mi_amax_scale. */
int f8mi_cast_dynamic(const void* x, int64_t rows, int64_t cols, int64_t ld, int in_dtype, int fp8_fmt, float* scale_dev,
                      uint8_t* out, int out_layout, uint8_t* out_t, int out_t_layout, void* workspace, void* stream);

/* f8mi_cast_dynamic without the workspace argument, for callers that cannot allocate device memory (code under HIP
 * graph capture, tight serving loops, harnesses that forbid hipMalloc) and so have no workspace to bring.  No
 * counterpart in the reference.  The per-workgroup partial maxima go to an array of F8MI_STATIC_SCRATCH_BYTES that is
 * part of the library's device code: every GPU the library runs on holds it from load until the process ends.  The
 * call allocates and frees nothing (the first call on a device looks the array's address up, once).  Same kernels,
 * same result bits as f8mi_cast_dynamic.  All calls on one GPU share the one array: calls that can overlap in time
 * on the same GPU (two streams, two host threads) race on it -- give such callers f8mi_cast_dynamic and a workspace
 * each.  The array keeps the last call's contents; nothing in it needs to start at zero.  Tensors of more than
 * F8MI_STATIC_MAX_ELEMS elements are refused with F8MI_ERR_INVALID_ARG.
 * The first call on a device asks the runtime for the array's address on the device that is current (which, as for
 * every entry point, must be the device `stream` belongs to); that query may load the library's code onto the device
 * and is not something to do while a stream is being captured.  Make one ordinary call on each device before the
 * first capture (any size will do); from then on the entry point only launches kernels and may be captured and
 * replayed. */
#define F8MI_STATIC_SCRATCH_BYTES 4096
#define F8MI_STATIC_MAX_ELEMS (1ll << 36)
int f8mi_cast_dynamic_static(const void* x, int64_t rows, int64_t cols, int64_t ld, int in_dtype, int fp8_fmt,
                             float* scale_dev, uint8_t* out, int out_layout, uint8_t* out_t, int out_t_layout,
                             void* stream);

/* f8mi_gemm_nt on k-blocked operands: a = [k/64][m][64], bt = [k/64][n][64], both 16-byte
 * aligned.  Needs k % 64 == 0 and k >= 384 (F8MI_ERR_UNSUPPORTED otherwise: keep such operands
 * row-major and call f8mi_gemm_nt).  Same arithmetic, same result bits as f8mi_gemm_nt. */
int f8mi_gemm_nt_kb(const void* a, int a_fmt, const void* bt, int b_fmt, int64_t m, int64_t n, int64_t k,
                    const float* scale_a_dev, const float* scale_b_dev, void* c, int c_dtype, int64_t ldc,
                    const void* bias_dev, void* stream);

/* f8mi_gemm_nt / f8mi_gemm_nt_kb with scratch memory for the library to use: `workspace` (16-byte aligned device
 * memory, `workspace_bytes` long, contents irrelevant before and after; calls sharing it must not overlap) lets an
 * output of few tiles with a long k be computed with k split over workgroups -- an inference linear with 17 to a few
 * hundred rows and a long contraction, which would otherwise leave most CUs idle: partial sums go to the workspace
 * and a second kernel adds them in a fixed order (deterministic; another summation order than without the split,
 * so the two agree within the accumulation tolerance, not bit for bit).  Which path runs depends on (m, n, k),
 * alignment and workspace_bytes only; F8MI_GEMM_WORKSPACE_BYTES is enough for every case that is ever split.
 * With workspace NULL they are f8mi_gemm_nt / f8mi_gemm_nt_kb.  No counterpart in the reference (torch._scaled_mm
 * hides hipBLASLt's own workspace, float8_python_api.py:24-64). */
#define F8MI_GEMM_WORKSPACE_BYTES (32ll << 20)
int f8mi_gemm_nt_ws(const void* a, int a_fmt, int64_t lda, const void* bt, int b_fmt, int64_t ldb, int64_t m,
                    int64_t n, int64_t k, const float* scale_a_dev, const float* scale_b_dev, void* c, int c_dtype,
                    int64_t ldc, const void* bias_dev, void* workspace, int64_t workspace_bytes, void* stream);
int f8mi_gemm_nt_kb_ws(const void* a, int a_fmt, const void* bt, int b_fmt, int64_t m, int64_t n, int64_t k,
                       const float* scale_a_dev, const float* scale_b_dev, void* c, int c_dtype, int64_t ldc,
                       const void* bias_dev, void* workspace, int64_t workspace_bytes, void* stream);

/* Which kernel f8mi_gemm_nt(_ws) / f8mi_gemm_nt_kb(_ws) would run for an m x n x k product (no GPU needed; for tests,
 * logs and benchmarks).  `aligned`: operands and row strides are 16-byte aligned (k-blocked operands always are);
 * workspace_bytes: 0 without a workspace.  Returns a F8MI_PLAN_* code in bits 0-7, the number of parts k is split
 * into in bits 8-15 and, where 128-row tiles take part, 1 (128 x 128) or 2 (128 x 256) in bits 16-23; 0 for an
 * empty product.  No counterpart in the reference. */
#define F8MI_PLAN_TILES128_SPLIT_K 1 /* 128-row tiles, k split over workgroups, second kernel adds the parts */
#define F8MI_PLAN_FEW_ROWS 2         /* Bt streamed once per 128 rows, k split over the waves of a workgroup */
#define F8MI_PLAN_TILES128 3         /* 128 x 128 or 128 x 256 tiles */
#define F8MI_PLAN_TILES256 4         /* 256 x 256 tiles, 16x16x128 MFMA, operands through LDS-DMA */
#define F8MI_PLAN_TILES256_AND_128 5 /* the same for the tile rows of whole rounds, 128-row tiles for the rest */
#define F8MI_PLAN_TILES256_MFMA32 6  /* 256 x 256 tiles, 32x32x64 MFMA (k % 128 == 64) */
#define F8MI_PLAN_STAGED 7           /* 256 x 256 tiles, register-staged (ragged or short k, unaligned operands) */
int f8mi_gemm_plan(int64_t m, int64_t n, int64_t k, int aligned, int64_t workspace_bytes);

/* f8mi_gemm_nt_kb with operands that may be given transposed, so that one k-blocked copy of a tensor serves
 * both GEMMs that use it (no transposed fp8 copies at all):
 *   a, a_transposed = 0: [k/64][m][64] as above;  = 1: [m/64][k][64], i.e. the matrix [k][m] k-blocked over m
 *   bt likewise with n.
 * Forward x*W^T takes (0, 0); grad_input dY*W takes a = dY8 [n_out/64][tokens][64] (0) and bt = the forward's
 * W8 [k_in/64][n_out][64] (1); grad_weight dY^T*x takes a = that dY8 (1) and bt = the forward's x8 (1).
 * (1, 0) is not built.  Transposed operands need k % 128 == 0, k >= 384 and the operand's row count (m or n)
 * to be a multiple of 64.  Same result bits as f8mi_gemm_nt on the row-major operands (for m > 256: the
 * few-row kernel of f8mi_gemm_nt is not used for transposed operands). */
int f8mi_gemm_kb_ex(const void* a, int a_fmt, int a_transposed, const void* bt, int b_fmt, int b_transposed, int64_t m,
                    int64_t n, int64_t k, const float* scale_a_dev, const float* scale_b_dev, void* c, int c_dtype,
                    int64_t ldc, const void* bias_dev, void* stream);

/* f8mi_gemm_nt on ROW-MAJOR fp8 operands either of which may be given transposed, so that the fp8 transposes
 * preprocess_addmm makes for torch._scaled_mm's layout rule (a row-major, b column-major: float8_ops.py:131-155, the
 * .t().contiguous().t() of :150-153) need not be made: the matrix-core kernel transposes on the way from LDS to the
 * registers.
 *   a, a_transposed = 0: [m][k], row stride lda >= k;  = 1: [k][m], row stride lda >= m (the memory of a.t())
 *   bt, b_transposed = 0: [n][k], row stride ldb >= k; = 1: [k][n], row stride ldb >= n (b of a @ b, row-major)
 * In the reference's words: forward x @ W.t() is (0, 0); grad_input dY @ W, W row-major, is (0, 1); grad_weight
 * dY.t() @ x, both row-major, is (1, 1).  (0, 0) is f8mi_gemm_nt.  Transposed operands are taken when k % 128 == 0,
 * k >= 384, the transposed operand's row count (n; m too for (1, 1)) is a multiple of 64, addresses and row strides
 * are 16-byte aligned and the output has more than 256 tiles of 128 x 128; otherwise, and for (1, 0), the call
 * returns F8MI_ERR_UNSUPPORTED without having launched anything and the caller makes the copy the reference makes.
 * Same result bits as f8mi_gemm_nt on the copies. */
int f8mi_gemm_ex(const void* a, int a_fmt, int a_transposed, int64_t lda, const void* bt, int b_fmt, int b_transposed, int64_t ldb,
                 int64_t m, int64_t n, int64_t k, const float* scale_a_dev, const float* scale_b_dev, void* c, int c_dtype,
                 int64_t ldc, const void* bias_dev, void* stream);

/* One (layer, tensor) row of the delayed-scaling bookkeeping; all device pointers. */
typedef struct f8mi_sync_entry {
    float* amax;    /* [1]        fp8_amax_*          */
    float* history; /* [hist_len] fp8_amax_history_*  */
    float* scale;   /* [1]        fp8_scale_*         */
    int64_t fp8_fmt;
} f8mi_sync_entry;

/*
 * For each of the n entries: S = roll(history, 1); S[0] = amax;
 * scale = fmax * (1 / clamp(max(S), 1e-12)) in fp32 (<= 65504 if orig_is_fp16).
 * Replaces the body of sync_float8_amax_and_scale_history
 * (float8_linear_utils.py:287-319: _update_history_stack :37-56 and
 * amax_history_to_scale_stack, float8_utils.py:80-99) in one launch.
 * writeback_history = 0 reproduces the reference, which rolls a stacked copy
 * and leaves each layer's history buffer untouched; 1 stores S back.
 * `entries_dev` is a device array of n f8mi_sync_entry.
 */
int f8mi_sync(const f8mi_sync_entry* entries_dev, int n, int hist_len, int orig_is_fp16, int writeback_history,
              void* stream);

/* f8mi_sync with the entries in HOST memory: they travel to the GPU by value, as kernel arguments, 32 per launch, so
 * there is no table in device memory to build, copy or keep alive.  For callers whose device allocations are managed
 * by someone else -- a compiled graph under torch.compile(mode="reduce-overhead") must not keep a tensor of its own
 * inside the graph's memory pool -- and for one-off calls.  Under stream capture the pointers are baked into the
 * captured launches: the buffers must stay where they are (as for any captured kernel). */
int f8mi_sync_host(const f8mi_sync_entry* entries_host, int n, int hist_len, int orig_is_fp16, int writeback_history,
                   void* stream);

/*
 * First-iteration initialisation of one tensor's buffers
 * (_maybe_initialize_amaxes_scales_for_float8_cast, float8_scaling_utils.py:99-125):
 * history[0] = *amax; *scale = fmax * (1 / clamp(max(history), 1e-12)).
 * `amax_dev` must already hold this step's amax (f8mi_amax_scale).
 */
int f8mi_delayed_init(const float* amax_dev, float* history_dev, float* scale_dev, int hist_len, int fp8_fmt,
                      int orig_is_fp16, void* stream);

/*
 * Optional per-kernel timing with HIP events on the launch stream.  While
 * enabled every launch of kernel class `kernel` (F8MI_K_*) is bracketed by two
 * events; f8mi_prof_read synchronises them and returns launches, summed
 * milliseconds and summed algorithmic work (bytes for amax/cast/sync, flop for
 * gemm).  Off by default; meant for benchmarks, not for training loops.
 */
int f8mi_prof_enable(int on);
int f8mi_prof_reset(void);
int f8mi_prof_read(int kernel, uint64_t* launches, double* total_ms, double* total_work);

#ifdef __cplusplus
}
#endif
#endif /* F8MI_H */
