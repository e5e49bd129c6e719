/*
 * hk_rowwise.h — C-ABI of the gfx950 (MI355X) device layer for Hetu's row-wise
 * operator kernels: LayerNorm / RMSNorm forward+backward, Softmax
 * forward+backward, fused SoftmaxCrossEntropy (sparse int64 labels and dense
 * labels) forward+backward, Reduce sum/mean over arbitrary axes, plus the
 * stream / event / memory calls the host-side wrappers need.
 *
 * Everything here is `extern "C"`, plain pointers and sizes.  All device
 * pointers are HIP device addresses on the current device; `hkStream_t` is a
 * `hipStream_t` (NULL = the null stream).  Every function returns HK_OK (0) or
 * a negative error code and never throws; `hk_last_error()` gives the message
 * of the calling thread's last failure.  Kernels are launched asynchronously
 * on the given stream; no entry point synchronises the device.
 *
 * dtype codes equal the numeric values of hetu::DataType
 * (hetu/core/dtype.h:9-22) so the C++ layer can pass them through.
 */
#ifndef HK_ROWWISE_H_
#define HK_ROWWISE_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define HK_API __attribute__((visibility("default")))

/* ---- error codes -------------------------------------------------------- */
enum {
  HK_OK = 0,
  HK_ERR_INVALID = -1,      /* bad argument (null pointer, negative size, bad axis ...) */
  HK_ERR_UNSUPPORTED = -2,  /* dtype / feature not implemented (HT_NOT_IMPLEMENTED upstream) */
  HK_ERR_HIP = -3,          /* a HIP runtime call failed */
  HK_ERR_WORKSPACE = -4     /* workspace missing or too small */
};

/* ---- dtype codes: hetu/core/dtype.h:9-22 -------------------------------- */
enum {
  HK_UINT8 = 0,
  HK_INT8 = 1,
  HK_INT16 = 2,
  HK_INT32 = 3,
  HK_INT64 = 4,
  HK_FLOAT16 = 5,
  HK_FLOAT32 = 6,
  HK_FLOAT64 = 7,
  HK_BFLOAT16 = 8,
  HK_BOOL = 9
};

/* ---- reduction codes: hetu/core/reduction_type.h:7-15 (kSUM, kMEAN) ------ */
/* values of hetu::ReductionType (hetu/core/reduction_type.h:7-15) */
enum { HK_REDUCE_SUM = 0, HK_REDUCE_MEAN = 1, HK_REDUCE_MAX = 2, HK_REDUCE_MIN = 3, HK_REDUCE_PROD = 4 };

/* second per-row statistic written/read by the LayerNorm entries */
enum {
  HK_STAT_VAR = 0,  /* biased variance   — LayerNormCuda,      LayerNorm.cu:43-50   */
  HK_STAT_RSTD = 1  /* 1/sqrt(var + eps) — FusedLayerNormCuda, FusedLayerNorm.cu:422 */
};

typedef struct ihipStream_t* hkStream_t;
typedef struct ihipEvent_t* hkEvent_t;

HK_API const char* hk_last_error(void);
HK_API const char* hk_version(void);

/* ======================================================================== *
 * Device / memory / stream / event layer.
 * Replaces the raw CUDA calls under hetu/impl/stream/CUDAStream.{h,cc},
 * hetu/impl/memory/CUDACachingMemoryPool.cu and hetu/impl/utils/cuda_utils.h.
 * ======================================================================== */
HK_API int hk_device_count(int* count);                 /* cuda_utils.h: GetDeviceCount      */
HK_API int hk_set_device(int device);                   /* cuda_utils.h:103-127 device guard  */
HK_API int hk_get_device(int* device);
HK_API int hk_device_sync(void);
HK_API int hk_mem_get_info(size_t* free_bytes, size_t* total_bytes);
HK_API int hk_device_cu_count(int device, int* cus);    /* Device::dprop().multiProcessorCount */
/* LDS bytes of one compute unit and the most one workgroup may ask for, as the device reports them
 * (Device::dprop().maxSharedMemoryPerMultiProcessor / sharedMemPerBlock) */
HK_API int hk_device_lds_bytes(int device, size_t* per_cu, size_t* per_block);

HK_API int hk_malloc(void** ptr, size_t bytes);         /* CUDACachingMemoryPool.cu: cudaMalloc */
HK_API int hk_free(void* ptr);
HK_API int hk_host_malloc(void** ptr, size_t bytes);    /* pinned host memory */
HK_API int hk_host_free(void* ptr);
HK_API int hk_memcpy_h2d(void* dst, const void* src, size_t bytes, hkStream_t stream);
HK_API int hk_memcpy_d2h(void* dst, const void* src, size_t bytes, hkStream_t stream);
HK_API int hk_memcpy_d2d(void* dst, const void* src, size_t bytes, hkStream_t stream);
/* fill with a byte value through a kernel (safe under graph capture) */
HK_API int hk_memset(void* dst, int value, size_t bytes, hkStream_t stream);

/* CUDAStream.cc:28-40 — non-blocking streams at default priority */
HK_API int hk_stream_create(hkStream_t* stream);
HK_API int hk_stream_destroy(hkStream_t stream);
HK_API int hk_stream_sync(hkStream_t stream);           /* CUDAStream.cc:62-64 */
HK_API int hk_stream_wait_event(hkStream_t stream, hkEvent_t event); /* CUDAEvent::Block */

/* CUDAStream.h:50-114 — CUDAEvent */
HK_API int hk_event_create(hkEvent_t* event, int enable_timing);
HK_API int hk_event_destroy(hkEvent_t event);
HK_API int hk_event_record(hkEvent_t event, hkStream_t stream);
HK_API int hk_event_sync(hkEvent_t event);
HK_API int hk_event_query(hkEvent_t event, int* done);
/* nanoseconds from `start` to `stop` (CUDAEvent::TimeSince, CUDAStream.h:96-109) */
HK_API int hk_event_elapsed_ns(hkEvent_t start, hkEvent_t stop, int64_t* ns);

/* Debugging / tuning hook, not part of the operator interface: launch-shape overrides for sweeps (bench.py,
 * profiling).  The values are process-wide (every device, every stream, every thread sees them; they are read
 * atomically) and change performance only, never results.  Key names are listed in hk_tune_keys(); value 0
 * restores the automatic choice.  A deployment leaves them alone. */
HK_API int hk_tune_set(const char* key, int value);
HK_API const char* hk_tune_keys(void);

/* Measurement hook: the next launch of an operator's main kernel (the one that
 * streams the rows; not the small fold / finalize launches) made by the calling
 * thread carries `before` and `after` on its own dispatch (hipExtLaunchKernelGGL),
 * so that hk_event_elapsed_ns(before, after) is that kernel's begin-to-end time on
 * its stream; then the hook clears itself.  Pass NULLs to cancel. */
HK_API int hk_profile_next_kernel(hkEvent_t before, hkEvent_t after);

/* Plain streaming copy kernel of `bytes` (multiple of 16, 16-byte aligned):
 * calibration reference for bandwidth counters and timings. */
HK_API int hk_copy_kernel(void* dst, const void* src, size_t bytes, hkStream_t stream);

/* Gathers a strided view into a dense row-major array (what the reference's
 * OffsetCalculator does per element, hetu/impl/utils/offset_calculator.cuh:16-68).
 * shape/strides in elements, ndim <= 8. */
HK_API int hk_strided_copy(int dtype, const void* src, void* dst, int ndim,
                           const int64_t* shape, const int64_t* src_strides,
                           hkStream_t stream);

/* The other direction: lays a dense row-major array over a strided view (the output side of the same
 * OffsetCalculator, offset_calculator.cuh:16-68: the reference's kernels write every element through it).
 * Used for an operator output that is neither dense nor row-pitched. */
HK_API int hk_strided_scatter(int dtype, const void* src, void* dst, int ndim,
                              const int64_t* shape, const int64_t* dst_strides,
                              hkStream_t stream);

/* ======================================================================== *
 * LayerNorm.
 * x, y: [rows, cols] dense, dtype `dtype` (fp32 / bf16 / fp16); gamma, beta:
 * [cols] same dtype (either may be NULL: gamma=1 / beta=0).
 * mean, stat: [rows] of `stats_dtype` (HK_FLOAT32 or `dtype`).
 *
 * Replaces LayerNormCuda (hetu/impl/kernel/LayerNorm.cu:66-121; stat_kind
 * HK_STAT_VAR, stats_dtype = dtype) and FusedLayerNormCuda
 * (hetu/impl/kernel/FusedLayerNorm.cu:967-1004; HK_STAT_RSTD, HK_FLOAT32).
 * ======================================================================== */
HK_API int hk_layer_norm_fwd(int dtype, const void* x, const void* gamma, const void* beta,
                             void* y, void* mean, void* stat, int stats_dtype, int stat_kind,
                             int64_t rows, int64_t cols, float eps, hkStream_t stream);

/* The same on rows that lie a fixed pitch apart: row r of x starts x_pitch ELEMENTS after row r - 1, likewise
 * y (x_pitch, y_pitch >= cols; pitch == cols is the dense call above).  This is the view a column slice
 * x[:, a:b] of a wider array, or a row-padded buffer, presents; the last dimension must have unit stride.
 * A pitch that is a whole number of 16-byte vectors keeps the 128-bit kernels; any other pitch is taken by
 * the element-wise fallback.  Replaces, for such views, the per-element StridedOffsetCalculator of the
 * reference (hetu/impl/utils/offset_calculator.cuh:16-68), which its LayerNorm operators run on because they
 * accept non-contiguous inputs (hetu/graph/ops/LayerNorm.h:78-80). */
HK_API int hk_layer_norm_fwd_pitched(int dtype, const void* x, int64_t x_pitch, const void* gamma,
                                     const void* beta, void* y, int64_t y_pitch, void* mean, void* stat,
                                     int stats_dtype, int stat_kind, int64_t rows, int64_t cols,
                                     float eps, hkStream_t stream);

/* The same on rows laid out on up to THREE LEVELS: what a view with permuted leading dimensions presents, e.g.
 * x.permute(0, 2, 1, 3) of a dense [B, H, S, D] array normalised over D.  Rows are numbered
 *   r = (i2 * level_rows[1] + i1) * level_rows[0] + i0,   0 <= i_k < level_rows[k]
 * (the view's own row-major order) and row r of an operand starts
 *   i0 * steps[0] + i1 * steps[1] + i2 * steps[2]   ELEMENTS
 * from its base, every operand with its own steps (the strides of the view's leading dimensions, merged where
 * neighbours step together; a dense operand is {cols, level_rows[0] * cols, level_rows[0] * level_rows[1] * cols});
 * mean / stat stay dense [rows] arrays indexed by r.  The last dimension must have unit stride.  The row kernels
 * run on a three-dimensional grid, one level per grid dimension, so such a view is read and written IN PLACE with
 * the 128-bit kernels (steps that are whole 16-byte vectors), no gather or scatter pass: the traffic is the dense
 * call's.  The launch walks the levels in the order of their steps, smallest first (neighbouring workgroups then
 * touch neighbouring memory whatever order the view numbers its rows in); results do not depend on that order.
 * Replaces, for such views, the per-element OffsetCalculator of the reference
 * (hetu/impl/utils/offset_calculator.cuh:16-68, .cu:31-65), on which its LayerNorm / Softmax operators run
 * because they accept non-contiguous inputs (hetu/graph/ops/LayerNorm.h:78-80, Softmax.h:52-54). */
HK_API int hk_layer_norm_fwd_strided_rows(int dtype, const void* x, const int64_t x_steps[3], const void* gamma,
                                          const void* beta, void* y, const int64_t y_steps[3], void* mean,
                                          void* stat, int stats_dtype, int stat_kind,
                                          const int64_t level_rows[3], int64_t cols, float eps,
                                          hkStream_t stream);

/* Bytes of scratch hk_layer_norm_bwd / hk_dropout_add_ln_bwd need for the
 * column-sum partials of dgamma / dbeta. */
HK_API int hk_norm_bwd_workspace_bytes(int dtype, int64_t rows, int64_t cols, size_t* bytes);

/* LayerNorm backward.  dy, x_or_y, dx: [rows, cols]; dgamma, dbeta: [cols] of
 * `dtype` (either may be NULL).  mean/stat as written by hk_layer_norm_fwd.
 *  memory_efficient = 0: x_or_y is the forward input x.
 *  memory_efficient = 1: x_or_y is the forward OUTPUT y and x_hat is recomputed
 *    as (y - beta) / clamp_by_magnitude(gamma, eps)  (FusedLayerNorm.cu:486-503).
 *  clamp_gamma: apply clamp_by_magnitude(gamma, eps) to gamma in dx, as
 *    cuComputeGradInput does unconditionally (FusedLayerNorm.cu:911-938).
 * Replaces LayerNormGradientCuda (LayerNorm.cu:235-337) and
 * FusedLayerNormGradientCuda (FusedLayerNorm.cu:1006-1144). */
HK_API int hk_layer_norm_bwd(int dtype, const void* dy, const void* x_or_y, const void* gamma,
                             const void* beta, const void* mean, const void* stat,
                             int stats_dtype, int stat_kind, void* dx, void* dgamma,
                             void* dbeta, int64_t rows, int64_t cols, float eps,
                             int memory_efficient, int clamp_gamma, void* workspace,
                             size_t workspace_bytes, hkStream_t stream);

/* hk_layer_norm_bwd on row-pitched dy, x_or_y and dx (see hk_layer_norm_fwd_pitched). */
HK_API int hk_layer_norm_bwd_pitched(int dtype, const void* dy, int64_t dy_pitch, const void* x_or_y,
                                     int64_t x_pitch, const void* gamma, const void* beta,
                                     const void* mean, const void* stat, int stats_dtype, int stat_kind,
                                     void* dx, int64_t dx_pitch, void* dgamma, void* dbeta, int64_t rows,
                                     int64_t cols, float eps, int memory_efficient, int clamp_gamma,
                                     void* workspace, size_t workspace_bytes, hkStream_t stream);

/* hk_layer_norm_bwd on operands whose rows lie on up to three levels (see hk_layer_norm_fwd_strided_rows); the
 * workspace is that of hk_norm_bwd_workspace_bytes for rows = the product of level_rows.  The walking kernel
 * splits each row number itself (two integer divisions per row and workgroup), in its general instance. */
HK_API int hk_layer_norm_bwd_strided_rows(int dtype, const void* dy, const int64_t dy_steps[3], const void* x_or_y,
                                          const int64_t x_steps[3], const void* gamma, const void* beta,
                                          const void* mean, const void* stat, int stats_dtype, int stat_kind,
                                          void* dx, const int64_t dx_steps[3], void* dgamma, void* dbeta,
                                          const int64_t level_rows[3], int64_t cols, float eps,
                                          int memory_efficient, int clamp_gamma, void* workspace,
                                          size_t workspace_bytes, hkStream_t stream);

/* ======================================================================== *
 * Dropout-add-LayerNorm / RMSNorm (flash-attention layer_norm path).
 * Replaces DropoutAddLnFwdCuda (hetu/impl/kernel/RMSNorm.cu:91-264) and
 * DropoutAddLnBwdCuda (RMSNorm.cu:266-470) for the configuration Hetu's
 * RMSNorm / LayerNorm modules use: dropout_p = 0, no rowscale / colscale /
 * subset.  x0: [rows, cols] `itype`; residual (optional, may be NULL): [rows,
 * cols] `rtype`; gamma, beta (beta optional): [cols] `wtype`; z: [rows, cols]
 * `itype`; x_out (optional): the pre-norm sum x0 + residual in `rtype`, written
 * when non-NULL; mu, rsigma: [rows] fp32.
 *   rs = rsqrt(m2/cols + eps + (is_rms ? mu^2 : 0)),  z = gamma*rs*(x - (is_rms?0:mu)) + beta
 *   (flash-attn csrc/layer_norm ln_fwd_kernels.cuh:155-177).
 * ======================================================================== */
HK_API int hk_dropout_add_ln_fwd(int itype, int rtype, int wtype, const void* x0,
                                 const void* residual, const void* gamma, const void* beta,
                                 void* z, void* x_out, void* mu, void* rsigma, int64_t rows,
                                 int64_t cols, float eps, int is_rms_norm, hkStream_t stream);

/* dz: [rows, cols] `itype`; dx_in (optional): upstream gradient of the
 * pre-norm sum (`rtype`), added to dx; x: [rows, cols] `rtype`; dx0: [rows,
 * cols] `itype`; dresidual (optional): `rtype`; dgamma, dbeta: [cols] `wtype`
 * (either may be NULL).  An RMSNorm layer has no bias and passes dbeta = NULL, as the reference's RMSNorm operator
 * does when it was given no beta (hetu/graph/ops/RMSNorm.cc:156): that call takes the instances that form no
 * column sums of dy; dbeta under is_rms_norm is computed all the same when asked for, by a more general and
 * slightly slower instance.  (ln_bwd_kernels.cuh:126-221, finalize :301-442) */
HK_API int hk_dropout_add_ln_bwd(int itype, int rtype, int wtype, const void* dz,
                                 const void* dx_in, const void* x, const void* mu,
                                 const void* rsigma, const void* gamma, void* dx0,
                                 void* dresidual, void* dgamma, void* dbeta, int64_t rows,
                                 int64_t cols, int is_rms_norm, void* workspace,
                                 size_t workspace_bytes, hkStream_t stream);

/* The two calls above on row-pitched arrays (see hk_layer_norm_fwd_pitched): every [rows, cols] operand
 * carries its own pitch in elements; the pitch of an absent optional operand is ignored. */
HK_API int hk_dropout_add_ln_fwd_pitched(int itype, int rtype, int wtype, const void* x0, int64_t x0_pitch,
                                         const void* residual, int64_t residual_pitch, const void* gamma,
                                         const void* beta, void* z, int64_t z_pitch, void* x_out,
                                         int64_t x_out_pitch, void* mu, void* rsigma, int64_t rows,
                                         int64_t cols, float eps, int is_rms_norm, hkStream_t stream);
HK_API int hk_dropout_add_ln_bwd_pitched(int itype, int rtype, int wtype, const void* dz, int64_t dz_pitch,
                                         const void* dx_in, int64_t dx_in_pitch, const void* x,
                                         int64_t x_pitch, const void* mu, const void* rsigma,
                                         const void* gamma, void* dx0, int64_t dx0_pitch, void* dresidual,
                                         int64_t dresidual_pitch, void* dgamma, void* dbeta, int64_t rows,
                                         int64_t cols, int is_rms_norm, void* workspace,
                                         size_t workspace_bytes, hkStream_t stream);

/* The same two calls on operands whose rows lie on up to three levels (see hk_layer_norm_fwd_strided_rows);
 * the steps of an absent optional operand may be NULL. */
HK_API int hk_dropout_add_ln_fwd_strided_rows(int itype, int rtype, int wtype, const void* x0,
                                              const int64_t x0_steps[3], const void* residual,
                                              const int64_t residual_steps[3], const void* gamma,
                                              const void* beta, void* z, const int64_t z_steps[3], void* x_out,
                                              const int64_t x_out_steps[3], void* mu, void* rsigma,
                                              const int64_t level_rows[3], int64_t cols, float eps,
                                              int is_rms_norm, hkStream_t stream);
HK_API int hk_dropout_add_ln_bwd_strided_rows(int itype, int rtype, int wtype, const void* dz,
                                              const int64_t dz_steps[3], const void* dx_in,
                                              const int64_t dx_in_steps[3], const void* x,
                                              const int64_t x_steps[3], const void* mu, const void* rsigma,
                                              const void* gamma, void* dx0, const int64_t dx0_steps[3],
                                              void* dresidual, const int64_t dresidual_steps[3], void* dgamma,
                                              void* dbeta, const int64_t level_rows[3], int64_t cols,
                                              int is_rms_norm, void* workspace, size_t workspace_bytes,
                                              hkStream_t stream);

/* hk_dropout_add_ln_bwd for callers that cannot allocate device memory and so have no workspace to
 * pass: code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.  It has no
 * counterpart in the reference (whose launcher allocates its partials itself, RMSNorm.cu:429-431).
 * Same arguments and results, bit for bit, as hk_dropout_add_ln_bwd; the column-sum partials go to a
 * 16 MiB array that is part of the library's code object (one copy per device the library is loaded
 * on, held until the process ends).  The call allocates and frees nothing.  16 MiB is what the widest
 * row the register kernel takes (8192 columns) needs on 256 persistent workgroups; a plan that needs
 * more (hk_norm_bwd_workspace_bytes > 16 MiB: a device with more compute units, or a raised
 * "norm_bwd_blocks") is refused with HK_ERR_WORKSPACE.  All calls on one device share the array: calls that overlap on one
 * device (different streams, or threads) race and must be ordered by the caller.  The first call on a device looks
 * the array's address up (hipGetSymbolAddress, once per device): make that call before a capture begins; calls
 * recorded after it replay like any other kernel launch. */
HK_API int hk_dropout_add_ln_bwd_static(int itype, int rtype, int wtype, const void* dz,
                                        const void* dx_in, const void* x, const void* mu,
                                        const void* rsigma, const void* gamma, void* dx0,
                                        void* dresidual, void* dgamma, void* dbeta, int64_t rows,
                                        int64_t cols, int is_rms_norm, hkStream_t stream);

/* ------------------------------------------------------------------------ *
 * The same interface with every feature of the flash-attention layer_norm
 * kernels the reference vendors: dropout, per-row and per-column scaling, row
 * subsets, mixed input / residual / weight types and the parallel-residual form
 * (two inputs, two affine outputs of one normalisation).  The parameter blocks
 * mirror layer_norm::FwdParams / BwdParams (flash-attn csrc/layer_norm ln.h:29-175),
 * which is what DropoutAddLnFwdCuda / DropoutAddLnBwdCuda (RMSNorm.cu:91-264,
 * 266-470) and DropoutAddLnParallelResidualFwdCuda / ...BwdCuda (RMSNorm.cu:474-826)
 * fill before calling the launcher.  Arithmetic: ln_fwd_kernels.cuh:97-182,
 * ln_bwd_kernels.cuh:93-221, ln_parallel_residual_{fwd,bwd}_kernels.cuh.
 *
 * Types.  itype: x0, x1, z, z1, rowscale, dz, dz1, dx0, dx1.  rtype: residual,
 * x, dx, dresidual.  wtype: gamma, beta, gamma1, beta1, colscale and their
 * gradients.  mu, rs: fp32.  dmask, dmask1: uint8.  x0_subset, z_subset: int32.
 * Accepted (wtype, itype, rtype), the combinations the reference registers
 * (ln_fwd_4096.cu:6-15): all equal (fp32 / fp16 / bf16); (fp32, 16-bit, fp32);
 * (16-bit, same 16-bit, fp32); (fp32, 16-bit, same 16-bit); (fp16, fp32, fp32).
 * cols must be a multiple of 8 and at most 8192 (RMSNorm.cu:187).  Data
 * pointers must be 16-byte aligned, dmask pointers 8-byte aligned.
 *
 * Shapes.  rows = rows of x / residual / mu / rs (the length of the subsets when
 * given).  Without subsets x0, dmask, z, dz, dx0 have `rows` rows.  With
 * subsets (both or neither): x0, dmask, dx0 have x0_numrows rows, z and dz have
 * z_numrows rows; x0_subset[r] / z_subset[r] are 1-based row numbers, 0 means
 * "row r reads no x0" / "row r writes no z"; numbers outside [0, numrows] are
 * treated as 0; rowscale is ignored and rowscale_const used instead
 * (ln_fwd_kernels.cuh:99).  The parallel form (x1, gamma1, z1, dz1, dx1 ...)
 * excludes rowscale, colscale and subsets.
 *
 * Dropout.  keep-mask bytes are written to dmask (dmask1 for x1) by the forward
 * and read back by the backward.  The mask is a pure function of (seed, offset,
 * element index e in x0): word e % 4 of Philox4x32-10 with key = seed and counter
 * = (2 * (e / 4) + (0 for x0, 1 for x1), offset), mapped to (0, 1] as
 * float(bits) * 2^-32 + 2^-33 and kept when <= 1 - dropout_p.  (The reference
 * keys its stream by the CUDA thread index of a grid sized from the SM count,
 * ln_fwd_kernels.cuh:66-73, so its mask depends on the device it runs on.)
 *
 * Optional pointers may be NULL.  x is written when non-NULL.  Gradients of the
 * weights are written when non-NULL; they need the workspace reported by
 * hk_dropout_add_ln_bwd_ex_workspace_bytes.
 * ------------------------------------------------------------------------ */
typedef struct hkDropoutAddLnFwdParams {
  int itype, rtype, wtype;
  int64_t rows, cols, x0_numrows, z_numrows;
  const void* x0;        /* [rows | x0_numrows, cols] itype */
  const void* x1;        /* parallel form: second input */
  const void* residual;  /* [rows, cols] rtype */
  const void* gamma;     /* [cols] wtype */
  const void* beta;
  const void* gamma1;    /* parallel form: second affine pair (NULL: one output) */
  const void* beta1;
  const void* rowscale;  /* [rows] itype */
  const void* colscale;  /* [cols] wtype */
  const int32_t* x0_subset;
  const int32_t* z_subset;
  void* z;               /* [rows | z_numrows, cols] itype */
  void* z1;
  void* x;               /* [rows, cols] rtype: the pre-norm sum */
  uint8_t* dmask;        /* x0's shape; required when dropout_p > 0 */
  uint8_t* dmask1;       /* required when dropout_p > 0 and x1 is given */
  float* mu;             /* [rows] */
  float* rs;             /* [rows] */
  float dropout_p, epsilon, rowscale_const;
  int is_rms_norm;
  uint64_t seed, offset;
} hkDropoutAddLnFwdParams;

typedef struct hkDropoutAddLnBwdParams {
  int itype, rtype, wtype;
  int64_t rows, cols, x0_numrows, z_numrows;
  const void* dz;        /* [rows | z_numrows, cols] itype */
  const void* dz1;       /* parallel form, with gamma1 */
  const void* dx;        /* [rows, cols] rtype: upstream gradient of the pre-norm sum */
  const void* x;         /* [rows, cols] rtype */
  const void* x0;        /* itype; required with colscale */
  const uint8_t* dmask;  /* required when dropout_p > 0 */
  const uint8_t* dmask1;
  const float* mu;
  const float* rs;
  const void* gamma;
  const void* gamma1;
  const void* rowscale;
  const void* colscale;
  const int32_t* x0_subset;
  const int32_t* z_subset;
  void* dx0;             /* [rows | x0_numrows, cols] itype */
  void* dx1;             /* parallel form: gradient of x1 */
  void* dresidual;       /* [rows, cols] rtype */
  void* dgamma;          /* [cols] wtype */
  void* dbeta;
  void* dgamma1;
  void* dbeta1;
  void* dcolscale;
  void* workspace;
  size_t workspace_bytes;
  float dropout_p, rowscale_const;
  int is_rms_norm;
} hkDropoutAddLnBwdParams;

HK_API int hk_dropout_add_ln_fwd_ex(const hkDropoutAddLnFwdParams* params, hkStream_t stream);
HK_API int hk_dropout_add_ln_bwd_ex_workspace_bytes(const hkDropoutAddLnBwdParams* params,
                                                    size_t* bytes);
HK_API int hk_dropout_add_ln_bwd_ex(const hkDropoutAddLnBwdParams* params, hkStream_t stream);

/* ======================================================================== *
 * Spatial batch normalisation of a dense NCHW array (x viewed as [N, C, HW]) in
 * training mode.  The reference calls cuDNN (>= 7) for this
 * (hetu/impl/kernel/BatchNorm.cu:8-83, 84-165: cudnnBatchNormalizationForwardTraining /
 * cudnnBatchNormalizationBackward, CUDNN_BATCHNORM_SPATIAL); cuDNN is not part of
 * the reference's sources, so the arithmetic here restates its documented one:
 *   mean_c, var_c over N, H, W (biased);  y = scale (x - mean) / sqrt(var + eps) + bias;
 *   running_mean = (1 - momentum) running_mean + momentum mean;
 *   running_var  = (1 - momentum) running_var  + momentum var * m / (m - 1)   (m = N*HW);
 *   save_mean = mean,  save_invstd = 1 / sqrt(var + eps)   (the reference names this output save_var);
 *   dscale = sum dy xhat,  dbias = sum dy,  dx = scale invstd (dy - dbias / m - xhat dscale / m).
 * scale, bias, running_*, save_*, dscale, dbias are fp32 for fp16 / bf16 data and of the data type otherwise
 * (BatchNorm.cu:55-70).  running_* and save_* may be NULL in the forward, dscale / dbias in the backward.
 * ======================================================================== */
HK_API int hk_batch_norm_workspace_bytes(int dtype, int64_t N, int64_t C, int64_t HW, size_t* bytes);
HK_API int hk_batch_norm_fwd(int dtype, const void* x, const void* scale, const void* bias, void* y,
                             double momentum, double eps, void* running_mean, void* running_var,
                             void* save_mean, void* save_invstd, int64_t N, int64_t C, int64_t HW,
                             void* workspace, size_t workspace_bytes, hkStream_t stream);
HK_API int hk_batch_norm_bwd(int dtype, const void* dy, const void* x, const void* scale, void* dx,
                             void* dscale, void* dbias, const void* save_mean, const void* save_invstd,
                             int64_t N, int64_t C, int64_t HW, void* workspace, size_t workspace_bytes,
                             hkStream_t stream);

/* ======================================================================== *
 * Softmax along one dimension of a dense array viewed as [outer, dim, inner].
 * Replaces SoftmaxCuda (hetu/impl/kernel/Softmax.cu:250-310) and
 * SoftmaxGradientCuda (Softmax.cu:364-404): dx = dy*y - y*sum(dy*y).
 * ======================================================================== */
HK_API int hk_softmax_fwd(int dtype, const void* x, void* y, int64_t outer, int64_t dim,
                          int64_t inner, hkStream_t stream);
HK_API int hk_softmax_bwd(int dtype, const void* y, const void* dy, void* dx, int64_t outer,
                          int64_t dim, int64_t inner, hkStream_t stream);

/* Last-dimension softmax of [rows, cols] arrays whose rows lie a pitch (in elements, >= cols) apart: column
 * slices of wider buffers, row-padded arrays.  A pitch that is a whole number of 16-byte vectors keeps the
 * 128-bit kernels.  SoftmaxOp accepts non-contiguous inputs (hetu/graph/ops/Softmax.h:52-54) and the
 * reference resolves them per element (hetu/impl/utils/offset_calculator.cuh:16-68). */
HK_API int hk_softmax_fwd_pitched(int dtype, const void* x, int64_t x_pitch, void* y, int64_t y_pitch,
                                  int64_t rows, int64_t cols, hkStream_t stream);
HK_API int hk_softmax_bwd_pitched(int dtype, const void* y, int64_t y_pitch, const void* dy, int64_t dy_pitch,
                                  void* dx, int64_t dx_pitch, int64_t rows, int64_t cols, hkStream_t stream);

/* Last-dimension softmax of operands whose rows lie on up to three levels (see hk_layer_norm_fwd_strided_rows):
 * a view with permuted leading dimensions is read and written in place.  Rows must be whole 16-byte vectors
 * (HK_ERR_UNSUPPORTED otherwise; the caller then gathers). */
HK_API int hk_softmax_fwd_strided_rows(int dtype, const void* x, const int64_t x_steps[3], void* y,
                                       const int64_t y_steps[3], const int64_t level_rows[3], int64_t cols,
                                       hkStream_t stream);
HK_API int hk_softmax_bwd_strided_rows(int dtype, const void* y, const int64_t y_steps[3], const void* dy,
                                       const int64_t dy_steps[3], void* dx, const int64_t dx_steps[3],
                                       const int64_t level_rows[3], int64_t cols, hkStream_t stream);

/* ======================================================================== *
 * Fused softmax cross-entropy, sparse int64 labels.
 * logits: [rows, cols]; labels: [rows] int64; loss: [rows] `dtype`.
 *   loss[r] = (labels[r] == ignored_index) ? 0 : logsumexp(x[r,:]) - x[r, labels[r]]
 * Replaces SoftmaxCrossEntropySparseCuda
 * (hetu/impl/kernel/SoftmaxCrossEntropySparse.cu:239-274).
 * ======================================================================== */
HK_API int hk_sce_sparse_fwd(int dtype, const void* logits, const int64_t* labels, void* loss,
                             int64_t rows, int64_t cols, int64_t ignored_index,
                             hkStream_t stream);
/* dlogits[r, c] = (softmax(x[r,:])[c] - [c == labels[r]]) * grad_loss[r]; rows
 * whose label equals ignored_index are written as zeros, as the CPU twin and
 * softmax_cross_entropy_sparse_gradient_kernel do
 * (SoftmaxCrossEntropySparse.cc:49-55, .cu:93-140).
 * Replaces SoftmaxCrossEntropySparseGradientCuda (.cu:276-318). */
HK_API int hk_sce_sparse_bwd(int dtype, const void* logits, const int64_t* labels,
                             const void* grad_loss, void* dlogits, int64_t rows, int64_t cols,
                             int64_t ignored_index, hkStream_t stream);

/* The two calls above on logits / dlogits whose rows lie a pitch (in elements, >= cols) apart, e.g. the
 * un-padded columns of a vocabulary padded to a multiple of the tensor-parallel degree. */
HK_API int hk_sce_sparse_fwd_pitched(int dtype, const void* logits, int64_t logits_pitch,
                                     const int64_t* labels, void* loss, int64_t rows, int64_t cols,
                                     int64_t ignored_index, hkStream_t stream);
HK_API int hk_sce_sparse_bwd_pitched(int dtype, const void* logits, int64_t logits_pitch,
                                     const int64_t* labels, const void* grad_loss, void* dlogits,
                                     int64_t dlogits_pitch, int64_t rows, int64_t cols,
                                     int64_t ignored_index, hkStream_t stream);

/* The same on logits / dlogits whose rows lie on up to three levels (see hk_layer_norm_fwd_strided_rows);
 * labels, loss and grad_loss stay dense [rows] arrays indexed by the row's number. */
HK_API int hk_sce_sparse_fwd_strided_rows(int dtype, const void* logits, const int64_t logits_steps[3],
                                          const int64_t* labels, void* loss, const int64_t level_rows[3],
                                          int64_t cols, int64_t ignored_index, hkStream_t stream);
HK_API int hk_sce_sparse_bwd_strided_rows(int dtype, const void* logits, const int64_t logits_steps[3],
                                          const int64_t* labels, const void* grad_loss, void* dlogits,
                                          const int64_t dlogits_steps[3], const int64_t level_rows[3],
                                          int64_t cols, int64_t ignored_index, hkStream_t stream);

/* The same with the gradient of a REDUCED loss: grad_output holds one value and every row uses
 * round_dtype(grad_output[0] * round_dtype(scale)) -- what BroadcastShapeMul(grad, 1/rows) into a [rows]
 * array followed by the call above computes, without that array (SCESGradOpImpl::DoCompute,
 * hetu/graph/ops/SoftmaxCrossEntropySparse.cc:64-85; scale 1 for reduction "sum"). */
HK_API int hk_sce_sparse_bwd_reduced(int dtype, const void* logits, const int64_t* labels,
                                     const void* grad_output, double scale, void* dlogits,
                                     int64_t rows, int64_t cols, int64_t ignored_index,
                                     hkStream_t stream);

/* Dense (soft / one-hot) labels of the logits' shape:
 *   loss[r] = -sum_c labels[r,c] * log_softmax(x[r,:])[c]
 *   dlogits = (softmax(x) - labels) * grad_loss[r]
 * Replaces SoftmaxCrossEntropyCuda / SoftmaxCrossEntropyGradientCuda
 * (hetu/impl/kernel/SoftmaxCrossEntropy.cu:13-73, 91-171). */
HK_API int hk_sce_dense_fwd(int dtype, const void* logits, const void* labels, void* loss,
                            int64_t rows, int64_t cols, hkStream_t stream);
HK_API int hk_sce_dense_bwd(int dtype, const void* logits, const void* labels,
                            const void* grad_loss, void* dlogits, int64_t rows, int64_t cols,
                            hkStream_t stream);

/* Dense labels, gradient of a reduced loss (SoftmaxCrossEntropyGradientOpImpl::DoCompute,
 * hetu/graph/ops/SoftmaxCrossEntropy.cc:59-80); see hk_sce_sparse_bwd_reduced. */
HK_API int hk_sce_dense_bwd_reduced(int dtype, const void* logits, const void* labels,
                                    const void* grad_output, double scale, void* dlogits,
                                    int64_t rows, int64_t cols, hkStream_t stream);

/* ======================================================================== *
 * Negative log-likelihood loss on log-probabilities, int64 class labels.
 *   loss[r] = -pred[r, labels[r]]                    (0 for a label outside [0, cols))
 *   out[r, c] = (c == labels[r]) ? -grad_loss[r] * cols : 0     (every element written once)
 * Replaces NLLLossCuda / NLLLossGradientCuda (hetu/impl/kernel/NLLLoss.cu:43-86,
 * :88-128; the "* cols" factor is the reference's, :39).
 * ======================================================================== */
HK_API int hk_nll_loss_fwd(int dtype, const void* pred, const int64_t* labels, void* loss,
                           int64_t rows, int64_t cols, hkStream_t stream);
HK_API int hk_nll_loss_bwd(int dtype, const int64_t* labels, const void* grad_loss, void* out,
                           int64_t rows, int64_t cols, hkStream_t stream);

/* ======================================================================== *
 * Local kernels of the vocabulary-parallel cross-entropy: this device holds the
 * columns [vocab_start, vocab_end) of the logits, [rows, cols] dense.
 *   gather: picked[r] = logits[r, labels[r] - vocab_start] when the label lies in
 *     the shard, else 0; a row whose label is ignored_index gets picked = 0 AND
 *     lse = 0; lse of every other row is left untouched (the caller has put
 *     log(sum(exp)) there).
 *   bwd: out[r, c] = (softmax[r, c] - [c == labels[r] - vocab_start]) * grad_loss[r];
 *     the column test is on unsigned 64-bit values, so labels outside the shard
 *     and negative labels match nothing; ignored rows are not special-cased (the
 *     caller zeroes their grad_loss).  out may alias softmax.
 * Replaces VocabParallelCrossEntropyCuda / VocabParallelCrossEntropyGradientCuda
 * (hetu/impl/kernel/VocabParallelCrossEntropyLoss.cu:14-64, 69-119).
 * ======================================================================== */
HK_API int hk_vocab_parallel_ce_gather(int dtype, const void* logits, const int64_t* labels,
                                       int64_t rows, int64_t cols, int64_t vocab_start,
                                       int64_t vocab_end, int64_t ignored_index, void* picked,
                                       void* lse, hkStream_t stream);
HK_API int hk_vocab_parallel_ce_bwd(int dtype, const void* softmax, const int64_t* labels,
                                    const void* grad_loss, void* out, int64_t rows, int64_t cols,
                                    int64_t vocab_start, hkStream_t stream);

/* The same loss in its fused form: the shard is read once in the forward and once in the backward, and no
 * softmax array is kept.  No counterpart in the reference, which composes the loss from eight launches
 * (hetu/graph/ops/VocabParallelCrossEntropyLoss.cc:51-108: max, subtract, exp, sum, divide, log, gather,
 * subtract) and stores softmax for the backward.
 *   stats:   per row of the shard, in ONE pass: stats[0][r] = max_c x, stats[1][r] = sum_c exp(x - max),
 *            stats[2][r] = x[r, labels[r] - vocab_start] when the label lies in the shard, else 0
 *            (fp32, [3, rows]); an ignored row is not read and gets (-inf, 0, 0).
 *   combine: stats of all shards, [nshards, 3, rows] as an all-gather leaves them ->
 *            lse[r] = log sum over the whole row (fp32), loss[r] = lse - picked (0 for an ignored row).
 *            Either output may be NULL.
 *   bwd_fused: out[r, c] = (exp(x[r, c] - lse[r]) - [c == labels[r] - vocab_start]) * grad_loss[r];
 *            an ignored row is written as zeros.  out may alias logits. */
HK_API int hk_vocab_parallel_ce_stats(int dtype, const void* logits, const int64_t* labels, float* stats,
                                      int64_t rows, int64_t cols, int64_t vocab_start,
                                      int64_t ignored_index, hkStream_t stream);
HK_API int hk_vocab_parallel_ce_combine(int loss_dtype, const float* stats, int nshards,
                                        const int64_t* labels, int64_t ignored_index, void* loss,
                                        float* lse, int64_t rows, hkStream_t stream);
HK_API int hk_vocab_parallel_ce_bwd_fused(int dtype, const void* logits, const int64_t* labels,
                                          const float* lse, const void* grad_loss, void* out,
                                          int64_t rows, int64_t cols, int64_t vocab_start,
                                          int64_t ignored_index, hkStream_t stream);

/* ======================================================================== *
 * Element-wise operators on dense arrays of fp32 / bf16 / fp16 / fp64 (16-bit
 * floats compute in fp32 and round once).  out may alias an input of its shape.
 *   hk_unary: exp, log, negate, sqrt.  Replaces ExpCuda, LogCuda, OppositeCuda,
 *     SqrtCuda (hetu/impl/kernel/Exp.cu:12-29, Log.cu, Opposite.cu, Sqrt.cu).
 *   hk_binary_const: x op c, or c op x when scalar_first != 0 (sub, div); the
 *     constant is first rounded to the array's type.  Replaces AddConstCuda,
 *     SubConstCuda (c - x), MulConstCuda, DivConstCuda (c / x)
 *     (hetu/impl/kernel/BinaryConst.cu:10-53).
 *   hk_binary: out = a op b with broadcasting.  out is dense with shape
 *     out_shape[ndim] (ndim <= 8); a_strides / b_strides are the operands'
 *     element strides aligned to out_shape, 0 along a broadcast dimension.
 *     Replaces AddElewiseCuda, SubElewiseCuda, MulElewiseCuda, DivElewiseCuda
 *     (hetu/impl/kernel/BinaryElewise.cu) and the launch_loop_kernel /
 *     vectorize_broadcast_loop_kernel family they run on (Vectorized.cuh).
 * The arithmetic (hk_binary, hk_binary_const), negation and hk_broadcast also take the integer
 * types uint8 / int8 / int16 / int32 / int64, as the reference dispatches them
 * (HT_DISPATCH_INTEGER_AND_FLOATING_TYPES, BinaryElewise.cu:332, BinaryConst.cu:16,
 * Opposite.cu:19): results wrap in the type, division truncates; exp / log / sqrt are
 * floating only (HK_ERR_UNSUPPORTED otherwise, as for bool).
 * ======================================================================== */
enum { HK_UNARY_EXP = 0, HK_UNARY_LOG = 1, HK_UNARY_NEG = 2, HK_UNARY_SQRT = 3 };
enum { HK_BINARY_ADD = 0, HK_BINARY_SUB = 1, HK_BINARY_MUL = 2, HK_BINARY_DIV = 3 };
HK_API int hk_unary(int op, int dtype, const void* in, void* out, int64_t numel, hkStream_t stream);
HK_API int hk_binary_const(int op, int dtype, const void* in, double scalar, int scalar_first,
                           void* out, int64_t numel, hkStream_t stream);
HK_API int hk_binary(int op, int dtype, const void* a, const void* b, void* out, int ndim,
                     const int64_t* out_shape, const int64_t* a_strides, const int64_t* b_strides,
                     hkStream_t stream);

/* out = in broadcast to out_shape (dense), optionally times `scalar` (rounded to `dtype` first, as
 * static_cast<spec_t>(const_value) does).  in_strides holds, per output dimension, the input's stride in
 * elements, 0 where the input is broadcast along that dimension; a strided input view is read in place.
 * The backward of Reduce sum / mean and of every reduced loss.
 * Replaces broadcast_shape_kernel / broadcast_shape_mul_kernel and their launchers BroadcastShapeCuda /
 * BroadcastShapeMulCuda (hetu/impl/kernel/BroadcastShape.cu:11-28, 30-99, 101-117, 119-186). */
HK_API int hk_broadcast(int dtype, const void* in, int multiply, double scalar, void* out, int ndim,
                        const int64_t* out_shape, const int64_t* in_strides, hkStream_t stream);

/* ======================================================================== *
 * Reduce sum / mean / max / min / product over a set of axes of a (possibly
 * strided) array.
 * shape / strides (in elements) describe the input; axes must already be
 * wrapped to [0, ndim), may be unsorted or repeated (sorted + de-duplicated
 * inside, hetu/impl/kernel/Reduce.cuh:765-768).  The output is written dense,
 * kept dims in their original order.  bf16 / fp16 accumulate in fp32; mean is
 * sum * (1.0f / reduce_num) (hetu/impl/kernel/ReduceMean.cu:9-33).
 * out_dtype may be HK_FLOAT32 for bf16 / fp16 input (ReduceSum.cu:28-37).
 * naxes = 0 writes the dense copy of the input; a reduced extent of 0 writes
 * the empty sum 0 (mean: NaN for floating types); no kept element, no write.
 * Max / min return a NaN once one has been seen and start from -inf / +inf (the
 * type's extremes for integers); the product starts from 1; an empty reduced
 * extent writes those identities (ReduceMax.cu:10-25, ReduceMin.cu:10-25,
 * ReduceProd.cu:8-24).  A widened fp32 output exists for sum, mean and product.
 * Replaces ReduceSumCuda / ReduceMeanCuda / ReduceMaxCuda / ReduceMinCuda /
 * ReduceProdCuda (ReduceSum.cu:25-42, ReduceMean.cu:35-55, ReduceMax.cu:28-41,
 * ReduceMin.cu:28-41, ReduceProd.cu:26-45) and launch_reduce_kernel
 * (Reduce.cuh:757-844).
 * ======================================================================== */
HK_API int hk_reduce_workspace_bytes(int in_dtype, int ndim, const int64_t* shape,
                                     const int64_t* strides, int naxes, const int64_t* axes,
                                     size_t* bytes);
HK_API int hk_reduce(int in_dtype, int out_dtype, const void* in, void* out, int ndim,
                     const int64_t* shape, const int64_t* strides, int naxes,
                     const int64_t* axes, int op, void* workspace, size_t workspace_bytes,
                     hkStream_t stream);

/* p-norm over one dimension, out = (sum_k |x|^p)^(1/p), p >= 1 an integer, floating types; the reduction
 * runs on hk_reduce's planner and kernels (same shape / strides / workspace rules, workspace from
 * hk_reduce_workspace_bytes with that one axis), accumulating in fp32 for the 16-bit types.
 * Replaces NormCuda (hetu/impl/kernel/Norm1.cu:99-133).
 * Gradient over the middle dimension of a dense [before, reduce_size, after] array; norm and grad are dense
 * [before, after]: p = 1: sign(x) g;  p = 2: g x / norm;  p > 2: x |x|^(p-2) g / norm^(p-1);  0 where norm == 0.
 * Replaces NormGradientCuda (Norm1.cu:135-186). */
HK_API int hk_norm(int dtype, const void* in, void* out, int ndim, const int64_t* shape,
                   const int64_t* strides, int64_t dim, int64_t p, void* workspace,
                   size_t workspace_bytes, hkStream_t stream);
HK_API int hk_norm_bwd(int dtype, const void* in, const void* norm, const void* grad, void* out,
                       int64_t before, int64_t reduce_size, int64_t after, int64_t p,
                       hkStream_t stream);

#ifdef __cplusplus
}
#endif

#endif /* HK_ROWWISE_H_ */
