/* C entry points over the C++ operator layer (libhetu_rowwise.so): the
 * `<Kernel>Cuda` functions declared in hetu/graph/ops/kernel_links.h of the
 * reference and the NDArray statics that dispatch to them, callable from any
 * language with a C FFI.  Arrays are described, not owned: every HtArray
 * borrows caller memory for the duration of the call.  A NULL HtArray pointer
 * stands for an undefined NDArray (an optional operand left out).
 *
 * Every function returns HT_OK or the kind of C++ exception the layer threw;
 * ht_last_error() holds its message (thread-local).
 */
#ifndef HETU_OPS_C_H_
#define HETU_OPS_C_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define HT_API __attribute__((visibility("default")))

enum {
  HT_OK = 0,
  HT_ERR_ASSERTION = 1,       /* hetu::assertion_error   (HT_ASSERT*)        */
  HT_ERR_NOT_IMPLEMENTED = 2, /* hetu::not_implemented   (HT_NOT_IMPLEMENTED) */
  HT_ERR_VALUE = 3,           /* hetu::value_error       (HT_VALUE_ERROR)     */
  HT_ERR_RUNTIME = 4,         /* hetu::runtime_error, HIP failures            */
  HT_ERR_BAD_ALLOC = 5,       /* hetu::bad_alloc                              */
  HT_ERR_OTHER = 6
};

enum { HT_DEVICE_CPU = 0, HT_DEVICE_ACCEL = 1 };   /* hetu::DeviceType kCPU / kCUDA */
enum { HT_RED_SUM = 0, HT_RED_MEAN = 1, HT_RED_MAX = 2, HT_RED_MIN = 3, HT_RED_PROD = 4, HT_RED_NONE = 5 };

#define HT_C_MAX_NDIM 8

typedef struct HtArray {
  void* data;
  int32_t dtype;                 /* hetu::DataType value (HK_FLOAT32 ...)      */
  int32_t ndim;
  int64_t shape[HT_C_MAX_NDIM];
  int64_t stride[HT_C_MAX_NDIM];   /* in elements                                 */
  int32_t device_type;           /* HT_DEVICE_*                                 */
  int32_t device_index;
} HtArray;

HT_API const char* ht_last_error(void);

/* ---- kernel entry points (one per `<Kernel>Cuda` symbol) ---- */
HT_API int ht_layer_norm(const HtArray* in, const HtArray* scale, const HtArray* bias, HtArray* mean,
                         HtArray* var, HtArray* out, int64_t reduce_dims, float eps, int stream_index);
HT_API int ht_layer_norm_gradient(const HtArray* out_grads, const HtArray* in, const HtArray* scale,
                                  HtArray* grad_in, HtArray* grad_scale, HtArray* grad_bias,
                                  const HtArray* mean, const HtArray* var, int64_t reduce_dims, float eps,
                                  int stream_index);
HT_API int ht_fused_layer_norm(const HtArray* in, const HtArray* scale, const HtArray* bias, HtArray* mean,
                               HtArray* invvar, HtArray* out, int64_t reduce_dims, float eps,
                               int stream_index);
HT_API int ht_fused_layer_norm_gradient(const HtArray* out_grads, const HtArray* x_or_y, const HtArray* scale,
                                        const HtArray* bias, HtArray* grad_in, HtArray* grad_scale,
                                        HtArray* grad_bias, const HtArray* mean, const HtArray* invvar,
                                        int64_t reduce_dims, float eps, int inplace, int stream_index);
/* DropoutAddLnFwdCuda / DropoutAddLnBwdCuda with their full argument lists (hetu/impl/kernel/RMSNorm.cu:91-110,
 * 266-292; the *_part outputs of the backward are internal scratch here).  Optional arrays may be NULL. */
HT_API int ht_dropout_add_ln_fwd(const HtArray* x0, const HtArray* residual, const HtArray* gamma,
                                 const HtArray* beta, const HtArray* rowscale, const HtArray* colscale,
                                 const HtArray* x0_subset, const HtArray* z_subset, HtArray* z, HtArray* x,
                                 HtArray* dmask, HtArray* mu, HtArray* rsigma, float dropout_p, float epsilon,
                                 float rowscale_const, int64_t z_numrows, int residual_in_fp32, int is_rms_norm,
                                 int stream_index);
HT_API int ht_dropout_add_ln_bwd(const HtArray* dz, const HtArray* dx, const HtArray* x, const HtArray* x0,
                                 const HtArray* dmask, const HtArray* mu, const HtArray* rsigma,
                                 const HtArray* gamma, const HtArray* rowscale, const HtArray* colscale,
                                 const HtArray* x0_subset, const HtArray* z_subset, HtArray* dx0,
                                 HtArray* dresidual, HtArray* dgamma, HtArray* dbeta, HtArray* dcolscale,
                                 float dropout_p, float rowscale_const, int64_t x0_numrows, int has_residual,
                                 int is_rms_norm, int stream_index);
/* DropoutAddLnParallelResidualFwdCuda / ...BwdCuda (RMSNorm.cu:474-493, 642-668) */
HT_API int ht_dropout_add_ln_parallel_residual_fwd(const HtArray* x0, const HtArray* x1, const HtArray* residual,
                                                   const HtArray* gamma0, const HtArray* beta0,
                                                   const HtArray* gamma1, const HtArray* beta1, HtArray* z0,
                                                   HtArray* z1, HtArray* x, HtArray* dmask0, HtArray* dmask1,
                                                   HtArray* mu, HtArray* rsigma, float dropout_p, float epsilon,
                                                   int residual_in_fp32, int is_rms_norm, int stream_index);
HT_API int ht_dropout_add_ln_parallel_residual_bwd(const HtArray* dz0, const HtArray* dz1, const HtArray* dx,
                                                   const HtArray* x, const HtArray* dmask0, const HtArray* dmask1,
                                                   const HtArray* mu, const HtArray* rsigma, const HtArray* gamma0,
                                                   const HtArray* gamma1, HtArray* dx0, HtArray* dx1,
                                                   HtArray* dresidual, HtArray* dgamma0, HtArray* dbeta0,
                                                   HtArray* dgamma1, HtArray* dbeta1, float dropout_p, int has_x1,
                                                   int has_residual, int is_rms_norm, int stream_index);
/* SetCPURandomSeed (hetu/impl/random/CPURandomState.cc:13-18): seeds the source of dropout seeds; 0 is ignored */
HT_API int ht_set_random_seed(uint64_t seed);
HT_API int ht_instance_norm(const HtArray* in, HtArray* mean, HtArray* var, HtArray* out, float eps,
                            int stream_index);
HT_API int ht_instance_norm_gradient(const HtArray* out_grads, const HtArray* in, HtArray* grad_in,
                                     const HtArray* mean, const HtArray* var, float eps, int stream_index);
HT_API int ht_softmax(const HtArray* in, HtArray* out, int64_t dim, int stream_index);
HT_API int ht_softmax_gradient(const HtArray* y, const HtArray* dy, HtArray* dx, int64_t dim, int stream_index);
HT_API int ht_softmax_cross_entropy(const HtArray* pred, const HtArray* label, HtArray* loss, int stream_index);
HT_API int ht_softmax_cross_entropy_gradient(const HtArray* pred, const HtArray* label, const HtArray* grad_loss,
                                             HtArray* out, int stream_index);
HT_API int ht_softmax_cross_entropy_sparse(const HtArray* pred, const HtArray* label, HtArray* loss,
                                           int64_t ignored_index, int stream_index);
HT_API int ht_softmax_cross_entropy_sparse_gradient(const HtArray* pred, const HtArray* label,
                                                    const HtArray* grad_loss, HtArray* out,
                                                    int64_t ignored_index, int stream_index);
HT_API int ht_nll_loss(const HtArray* pred, const HtArray* label, HtArray* loss, int stream_index);
HT_API int ht_nll_loss_gradient(const HtArray* pred, const HtArray* label, const HtArray* grad_loss,
                                HtArray* out, int stream_index);
HT_API int ht_reduce(const HtArray* in, HtArray* out, const int64_t* axes, int naxes, int red_type,
                     int stream_index);

/* ---- NDArray statics: device dispatch + output allocation from the pool ----
 * `out` (and mean / var) describe caller memory the result is written to. */
/* Element-wise family.  op: 0 add, 1 sub, 2 mul, 3 div (binary); 0 exp, 1 log, 2 negate, 3 sqrt (unary).
 * ht_binary      -> AddElewiseCuda / SubElewiseCuda / MulElewiseCuda / DivElewiseCuda (BinaryElewise.cu)
 * ht_binary_const -> AddConstCuda / SubConstCuda (value - x) / MulConstCuda / DivConstCuda (value / x) (BinaryConst.cu)
 * ht_unary       -> ExpCuda / LogCuda / OppositeCuda / SqrtCuda
 * ht_ndarray_binary / _unary: NDArray::add / sub / mul / div / exp / log / neg / sqrt, which allocate their result
 * from the pool (copied into `out`); with in_place != 0 the first operand is passed as the output, as the
 * reference's loss op does (VocabParallelCrossEntropyLoss.cc:77-81). */
HT_API int ht_binary(int op, const HtArray* a, const HtArray* b, HtArray* out, int stream_index);
HT_API int ht_binary_const(int op, const HtArray* in, double value, HtArray* out, int stream_index);
HT_API int ht_unary(int op, const HtArray* in, HtArray* out, int stream_index);
HT_API int ht_ndarray_binary(int op, const HtArray* a, const HtArray* b, HtArray* out, int in_place,
                             int stream_index);
HT_API int ht_ndarray_unary(int op, const HtArray* in, HtArray* out, int in_place, int stream_index);
/* BatchNormCuda / BatchNormGradientCuda (hetu/impl/kernel/BatchNorm.cu:8-83, 84-165) */
HT_API int ht_batch_norm(const HtArray* input_X, const HtArray* bn_scale, const HtArray* bn_bias, HtArray* output_Y,
                         double momentum, double eps, HtArray* running_mean, HtArray* running_var,
                         HtArray* save_mean, HtArray* save_var, int stream_index);
HT_API int ht_batch_norm_gradient(const HtArray* gradient_Y, const HtArray* input_X, const HtArray* bn_scale,
                                  HtArray* gradient_X, HtArray* gradient_bn_scale, HtArray* gradient_bn_bias,
                                  double eps, HtArray* save_mean, HtArray* save_var, int stream_index);
/* NormCuda / NormGradientCuda (hetu/impl/kernel/Norm1.cu:99-186) and NDArray::norm (result copied into `out`) */
HT_API int ht_norm(const HtArray* input, HtArray* output, int64_t dim, int64_t p, int stream_index);
HT_API int ht_norm_gradient(const HtArray* input, const HtArray* output, const HtArray* output_grad,
                            HtArray* input_grad, int64_t dim, int64_t p, int stream_index);
HT_API int ht_ndarray_norm(const HtArray* input, int64_t p, int64_t dim, int keepdim, HtArray* out,
                           int stream_index);
/* VocabParallelCrossEntropyCuda / VocabParallelCrossEntropyGradientCuda
 * (hetu/impl/kernel/VocabParallelCrossEntropyLoss.cu:38-64, 94-119) */
HT_API int ht_vocab_parallel_cross_entropy(const HtArray* vocab_parallel_logits, const HtArray* labels,
                                           int64_t vocab_start_index, int64_t vocab_end_index,
                                           int64_t ignored_index, HtArray* predicted_logits_partial,
                                           HtArray* log_sum_exp_logits, int stream_index);
HT_API int ht_vocab_parallel_cross_entropy_gradient(const HtArray* softmax, const HtArray* labels,
                                                    int64_t vocab_start_index, int64_t vocab_end_index,
                                                    int64_t ignored_index, const HtArray* grad_loss,
                                                    HtArray* output, int stream_index);
HT_API int ht_ndarray_reduce(const HtArray* in, int red_type, const int64_t* axes, int naxes, int keepdims,
                             HtArray* out, int stream_index);
HT_API int ht_ndarray_softmax(const HtArray* in, int64_t dim, HtArray* out, int stream_index);
HT_API int ht_ndarray_layernorm(const HtArray* in, const HtArray* scale, const HtArray* bias,
                                int normalized_ndim, double eps, int fused, HtArray* out, HtArray* mean,
                                HtArray* var, int stream_index);
/* sparse = 1: int64 labels + ignored_index; sparse = 0: dense labels. */
HT_API int ht_ndarray_sceloss(const HtArray* preds, const HtArray* labels, int sparse, int64_t ignored_index,
                              int reduction, HtArray* out, int stream_index);

/* ---- gradients of the reductions and of the reduced losses ---- */
/* BroadcastShapeCuda / BroadcastShapeMulCuda (hetu/impl/kernel/BroadcastShape.cu:30-99, 119-186);
 * multiply = 0 ignores const_value. */
HT_API int ht_broadcast_shape(const HtArray* input, int multiply, double const_value, HtArray* output,
                              const int64_t* add_axes, int n_add_axes, int stream_index);
/* ReduceGradientOpImpl::DoCompute (hetu/graph/ops/Reduce.cc:153-165): output has the reduced input's shape;
 * keepdims holds n_keepdims (= naxes, or 1 for all) flags. */
HT_API int ht_reduce_gradient(const HtArray* grad_output, int reduction, const int64_t* axes, int naxes,
                              const int* keepdims, int n_keepdims, HtArray* output, int stream_index);
/* SCESGradOpImpl / SCEGradOpImpl::DoCompute (hetu/graph/ops/SoftmaxCrossEntropySparse.cc:64-85,
 * SoftmaxCrossEntropy.cc:59-80).  sparse as in ht_ndarray_sceloss; fused = 0 runs the reference's two steps
 * (broadcast, then the gradient kernel), 1 the single kernel that takes the one gradient value. */
HT_API int ht_sceloss_gradient(const HtArray* preds, const HtArray* labels, const HtArray* grad_output, int sparse,
                               int64_t ignored_index, int reduction, int fused, HtArray* output,
                               int stream_index);

/* ---- streams and the device memory pool ---- */
HT_API int ht_stream_sync(int device_index, int stream_index);
HT_API int ht_synchronize_all(void);
/* Host streams (Device(kCPU), index 1..15) are task queues with one worker thread each, as in
 * hetu/impl/stream/CPUStream.cc:15-48 of the reference; index 0 runs in the calling thread.  Arrays handed to this C
 * face are borrowed, so by default every call on host arrays has finished when it returns.  ht_set_host_async(1)
 * makes host calls return as soon as their work is on its stream; the caller then keeps the buffers alive and
 * unchanged until ht_host_stream_sync (or ht_synchronize_all), which also reports a failure of such work.  Returns
 * the previous setting. */
HT_API int ht_set_host_async(int on);
HT_API int ht_host_stream_sync(int stream_index);
/* OpenMP team size of the host twins (the ...Cpu kernels), whichever thread runs them; threads <= 0 goes back to
 * the OpenMP runtime's default.  Returns the team size now in force.  For the CPU baseline legs of the benchmark
 * (all threads / one thread). */
HT_API int ht_set_host_threads(int threads);
HT_API int ht_pool_alloc(int device_index, size_t bytes, int stream_index, void** ptr, uint64_t* id,
                         size_t* granted_bytes);
HT_API int ht_pool_free(int device_index, void* ptr, uint64_t id, size_t granted_bytes);
HT_API int ht_pool_mark_used(int device_index, void* ptr, uint64_t id, size_t granted_bytes, int stream_index);
HT_API int ht_pool_empty_cache(int device_index);
/* allocated, peak_allocated, reserved, peak_reserved, alloc_cnt, free_cnt,
 * mark_cnt, segment_allocs, segment_frees, cache_hits, cross_stream_takes,
 * parked, splits, merges: 14 values */
HT_API int ht_pool_stats(int device_index, uint64_t* values, int n_values);

#ifdef __cplusplus
}
#endif

#endif /* HETU_OPS_C_H_ */
