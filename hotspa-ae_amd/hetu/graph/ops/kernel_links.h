// Declarations of the kernel entry points of the row-wise operator path and the
// device switch that picks them (hetu/graph/ops/kernel_links.h:12-21, 125-135,
// 168-175, 185-189, 199-206, 239-243, 260-269, 296-308, 362-397 of the reference).  The names
// `KERNEL##Cuda` / `KERNEL##Cpu` are produced by token pasting in the dispatch
// macros, so they are the link contract; the `Cuda` entries here are the
// gfx950 implementations.
#pragma once

#include "hetu/core/ndarray.h"
#include "hetu/core/stream.h"

namespace hetu {
namespace impl {

#define DECLARE_KERNEL(KERNEL, DEVICE, ...) extern void KERNEL##DEVICE(__VA_ARGS__)
#define DECLARE_KERNEL_CPU(KERNEL, ...) DECLARE_KERNEL(KERNEL, Cpu, __VA_ARGS__)
#define DECLARE_KERNEL_CUDA(KERNEL, ...) DECLARE_KERNEL(KERNEL, Cuda, __VA_ARGS__)
#define DECLARE_KERNEL_CPU_AND_CUDA(KERNEL, ...)                                                    \
  DECLARE_KERNEL_CPU(KERNEL, __VA_ARGS__);                                                          \
  DECLARE_KERNEL_CUDA(KERNEL, __VA_ARGS__)

// x0, residual_, gamma, beta_, rowscale_, colscale_, x0_subset_, z_subset_, z, x, dmask, mu, rsigma,
// dropout_p, epsilon, rowscale_const, z_numrows, residual_in_fp32, is_rms_norm
DECLARE_KERNEL_CUDA(DropoutAddLnFwd, const NDArray&, const NDArray&, const NDArray&, const NDArray&,
                    const NDArray&, const NDArray&, const NDArray&, const NDArray&, NDArray&, NDArray&, NDArray&,
                    NDArray&, NDArray&, const float, const float, const float, const int64_t, bool, bool,
                    const Stream&);
// dz, dx_, x, x0_, dmask_, mu, rsigma, gamma, rowscale_, colscale_, x0_subset_, z_subset_, dx0, dresidual,
// dgamma, dbeta, dgamma_part, dbeta_part, dcolscale, dcolscale_part, dropout_p, rowscale_const,
// x0_numrows, has_residual, is_rms_norm
DECLARE_KERNEL_CUDA(DropoutAddLnBwd, const NDArray&, const NDArray&, const NDArray&, const NDArray&,
                    const NDArray&, const NDArray&, const NDArray&, const NDArray&, const NDArray&, const NDArray&,
                    const NDArray&, const NDArray&, NDArray&, NDArray&, NDArray&, NDArray&, NDArray&, NDArray&,
                    NDArray&, NDArray&, const float, const float, const int64_t, const bool, bool, const Stream&);
// x0, x1_, residual_, gamma0, beta0_, gamma1_, beta1_, z0, z1, x, dmask0, dmask1, mu, rsigma, dropout_p,
// epsilon, residual_in_fp32, is_rms_norm
DECLARE_KERNEL_CUDA(DropoutAddLnParallelResidualFwd, const NDArray&, const NDArray&, const NDArray&,
                    const NDArray&, const NDArray&, const NDArray&, const NDArray&, NDArray&, NDArray&, NDArray&,
                    NDArray&, NDArray&, NDArray&, NDArray&, const float, const float, bool, bool, const Stream&);
// dz0, dz1_, dx_, x, dmask0_, dmask1_, mu, rsigma, gamma0, gamma1_, dx0, dx1, dresidual, dgamma0, dbeta0,
// dgamma1, dbeta1, dgamma0_part, dbeta0_part, dgamma1_part, dbeta1_part, dropout_p, has_x1, has_residual,
// is_rms_norm
DECLARE_KERNEL_CUDA(DropoutAddLnParallelResidualBwd, const NDArray&, const NDArray&, const NDArray&,
                    const NDArray&, const NDArray&, const NDArray&, const NDArray&, const NDArray&, const NDArray&,
                    const NDArray&, NDArray&, NDArray&, NDArray&, NDArray&, NDArray&, NDArray&, NDArray&, NDArray&,
                    NDArray&, NDArray&, NDArray&, const float, const bool, const bool, bool, const Stream&);
// in, scale, bias, mean, invvar, out, reduce_dims, eps
DECLARE_KERNEL_CUDA(FusedLayerNorm, const NDArray&, const NDArray&, const NDArray&, NDArray&, NDArray&, NDArray&,
                    int64_t, float, const Stream&);
// dy, x_or_y, scale, bias, dx, dscale, dbias, mean, invvar, reduce_dims, eps, inplace
DECLARE_KERNEL_CUDA(FusedLayerNormGradient, const NDArray&, const NDArray&, const NDArray&, const NDArray&,
                    NDArray&, NDArray&, NDArray&, const NDArray&, const NDArray&, int64_t, float, bool,
                    const Stream&);
// in, mean, var, out, eps   /   out_grads, in, grad_in, mean, var, eps
DECLARE_KERNEL_CPU_AND_CUDA(InstanceNorm, const NDArray&, NDArray&, NDArray&, NDArray&, float, const Stream&);
DECLARE_KERNEL_CPU_AND_CUDA(InstanceNormGradient, const NDArray&, const NDArray&, NDArray&, const NDArray&,
                            const NDArray&, float, const Stream&);
// in, scale, bias, mean, var, out, reduce_dims, eps
DECLARE_KERNEL_CPU_AND_CUDA(LayerNorm, const NDArray&, const NDArray&, const NDArray&, NDArray&, NDArray&,
                            NDArray&, int64_t, float, const Stream&);
// dy, x, scale, dx, dscale, dbias, mean, var, reduce_dims, eps
DECLARE_KERNEL_CPU_AND_CUDA(LayerNormGradient, const NDArray&, const NDArray&, const NDArray&, NDArray&, NDArray&,
                            NDArray&, const NDArray&, const NDArray&, int64_t, float, const Stream&);
// pred, label, loss   /   pred, label, grad_loss, output
DECLARE_KERNEL_CPU_AND_CUDA(NLLLoss, const NDArray&, const NDArray&, NDArray&, const Stream&);
DECLARE_KERNEL_CPU_AND_CUDA(NLLLossGradient, const NDArray&, const NDArray&, const NDArray&, NDArray&,
                            const Stream&);
DECLARE_KERNEL_CPU_AND_CUDA(Reduce, const NDArray&, NDArray&, const HTAxes&, ReductionType, const Stream&);
DECLARE_KERNEL_CPU_AND_CUDA(ReduceMean, const NDArray&, NDArray&, const int64_t*, int64_t, const Stream&);
DECLARE_KERNEL_CPU_AND_CUDA(ReduceSum, const NDArray&, NDArray&, const int64_t*, int64_t, const Stream&);
DECLARE_KERNEL_CPU_AND_CUDA(ReduceMax, const NDArray&, NDArray&, const int64_t*, int64_t, const Stream&);
DECLARE_KERNEL_CPU_AND_CUDA(ReduceMin, const NDArray&, NDArray&, const int64_t*, int64_t, const Stream&);
DECLARE_KERNEL_CPU_AND_CUDA(ReduceProd, const NDArray&, NDArray&, const int64_t*, int64_t, const Stream&);
// element-wise family (kernel_links.h:29-32, 117-120, 158, 214, 235-238, 250, 309-313 of the reference)
DECLARE_KERNEL_CPU_AND_CUDA(AddConst, const NDArray&, double, NDArray&, const Stream&);
DECLARE_KERNEL_CPU_AND_CUDA(SubConst, const NDArray&, double, NDArray&, const Stream&);
DECLARE_KERNEL_CPU_AND_CUDA(MulConst, const NDArray&, double, NDArray&, const Stream&);
DECLARE_KERNEL_CPU_AND_CUDA(DivConst, const NDArray&, double, NDArray&, const Stream&);
DECLARE_KERNEL_CPU_AND_CUDA(AddElewise, const NDArray&, const NDArray&, NDArray&, const Stream&);
DECLARE_KERNEL_CPU_AND_CUDA(SubElewise, const NDArray&, const NDArray&, NDArray&, const Stream&);
DECLARE_KERNEL_CPU_AND_CUDA(MulElewise, const NDArray&, const NDArray&, NDArray&, const Stream&);
DECLARE_KERNEL_CPU_AND_CUDA(DivElewise, const NDArray&, const NDArray&, NDArray&, const Stream&);
DECLARE_KERNEL_CPU_AND_CUDA(Exp, const NDArray&, NDArray&, const Stream&);
DECLARE_KERNEL_CPU_AND_CUDA(Log, const NDArray&, NDArray&, const Stream&);
DECLARE_KERNEL_CPU_AND_CUDA(Opposite, const NDArray&, NDArray&, const Stream&);
DECLARE_KERNEL_CPU_AND_CUDA(Sqrt, const NDArray&, NDArray&, const Stream&);
// input_X, bn_scale, bn_bias, output_Y, momentum, eps, running_mean, running_var, save_mean, save_var
DECLARE_KERNEL_CPU_AND_CUDA(BatchNorm, const NDArray&, const NDArray&, const NDArray&, NDArray&, double, double,
                            NDArray&, NDArray&, NDArray&, NDArray&, const Stream&);
// gradient_Y, input_X, bn_scale, gradient_X, gradient_bn_scale, gradient_bn_bias, eps, save_mean, save_var
DECLARE_KERNEL_CPU_AND_CUDA(BatchNormGradient, const NDArray&, const NDArray&, const NDArray&, NDArray&, NDArray&,
                            NDArray&, double, NDArray&, NDArray&, const Stream&);
// input, output, dim, p  /  input, output (the norm), output_grad, input_grad, dim, p   (kernel_links.h:244-247)
DECLARE_KERNEL_CPU_AND_CUDA(Norm, const NDArray&, NDArray&, int64_t, int64_t, const Stream&);
DECLARE_KERNEL_CPU_AND_CUDA(NormGradient, const NDArray&, const NDArray&, const NDArray&, NDArray&, int64_t, int64_t,
                            const Stream&);
// vocab_parallel_logits, labels, vocab_start_index, vocab_end_index, ignored_index, predicted_logits_partial,
// log_sum_exp_logits
DECLARE_KERNEL_CUDA(VocabParallelCrossEntropy, const NDArray&, const NDArray&, const int64_t, const int64_t,
                    const int64_t, NDArray&, NDArray&, const Stream&);
// softmax, labels, vocab_start_index, vocab_end_index, ignored_index, grad_loss, output
DECLARE_KERNEL_CUDA(VocabParallelCrossEntropyGradient, const NDArray&, const NDArray&, const int64_t, const int64_t,
                    const int64_t, const NDArray&, NDArray&, const Stream&);
DECLARE_KERNEL_CPU_AND_CUDA(Softmax, const NDArray&, NDArray&, int64_t, const Stream&);
// y, dy, dx, dim
DECLARE_KERNEL_CPU_AND_CUDA(SoftmaxGradient, const NDArray&, const NDArray&, NDArray&, int64_t, const Stream&);
DECLARE_KERNEL_CPU_AND_CUDA(SoftmaxCrossEntropy, const NDArray&, const NDArray&, NDArray&, const Stream&);
DECLARE_KERNEL_CPU_AND_CUDA(SoftmaxCrossEntropyGradient, const NDArray&, const NDArray&, const NDArray&, NDArray&,
                            const Stream&);
// pred, label, loss, ignored_index
DECLARE_KERNEL_CPU_AND_CUDA(SoftmaxCrossEntropySparse, const NDArray&, const NDArray&, NDArray&, const int64_t,
                            const Stream&);
// pred, label, grad_loss, output, ignored_index
DECLARE_KERNEL_CPU_AND_CUDA(SoftmaxCrossEntropySparseGradient, const NDArray&, const NDArray&, const NDArray&,
                            NDArray&, const int64_t, const Stream&);

#define HT_DISPATCH_KERNEL_CASE_CPU(KERNEL, ...)                                                    \
  case kCPU: {                                                                                      \
    KERNEL##Cpu(__VA_ARGS__);                                                                       \
    break;                                                                                          \
  }
#define HT_DISPATCH_KERNEL_CASE_CUDA(KERNEL, ...)                                                   \
  case kCUDA: {                                                                                     \
    KERNEL##Cuda(__VA_ARGS__);                                                                      \
    break;                                                                                          \
  }
#define HT_DISPATCH_KERNEL_SWITCH(DEVICE_TYPE, OP_TYPE, ...)                                        \
  do {                                                                                              \
    const auto& _device_type = DEVICE_TYPE;                                                         \
    switch (_device_type) {                                                                         \
      __VA_ARGS__                                                                                   \
      default:                                                                                      \
        HT_NOT_IMPLEMENTED << "\"" << OP_TYPE << "\" is not implemented for \""                     \
                           << DeviceType2Str(_device_type) << "\"";                                 \
    }                                                                                               \
  } while (0)
#define HT_DISPATCH_KERNEL_CPU_AND_CUDA(DEVICE_TYPE, OP_TYPE, KERNEL, ...)                          \
  HT_DISPATCH_KERNEL_SWITCH(DEVICE_TYPE, OP_TYPE,                                                   \
                            HT_DISPATCH_KERNEL_CASE_CPU(KERNEL, __VA_ARGS__)                        \
                              HT_DISPATCH_KERNEL_CASE_CUDA(KERNEL, __VA_ARGS__))
#define HT_DISPATCH_KERNEL_CPU_ONLY(DEVICE_TYPE, OP_TYPE, KERNEL, ...)                              \
  HT_DISPATCH_KERNEL_SWITCH(DEVICE_TYPE, OP_TYPE, HT_DISPATCH_KERNEL_CASE_CPU(KERNEL, __VA_ARGS__))
#define HT_DISPATCH_KERNEL_CUDA_ONLY(DEVICE_TYPE, OP_TYPE, KERNEL, ...)                             \
  HT_DISPATCH_KERNEL_SWITCH(DEVICE_TYPE, OP_TYPE, HT_DISPATCH_KERNEL_CASE_CUDA(KERNEL, __VA_ARGS__))

// input, output, add_axes  /  input, const_value, output, add_axes   (hetu/graph/ops/kernel_links.h:64-67)
DECLARE_KERNEL_CPU_AND_CUDA(BroadcastShape, const NDArray&, NDArray&, const HTShape&, const Stream&);
DECLARE_KERNEL_CPU_AND_CUDA(BroadcastShapeMul, const NDArray&, double, NDArray&, const HTShape&, const Stream&);
// The cross-entropy gradients fed the ONE gradient value of a reduced loss and its scale instead of a
// per-row array (no counterpart in the reference): pred, label, grad_output, scale, output, [ignored_index]
DECLARE_KERNEL_CUDA(SoftmaxCrossEntropySparseGradientReduced, const NDArray&, const NDArray&, const NDArray&, double,
                    NDArray&, const int64_t, const Stream&);
DECLARE_KERNEL_CUDA(SoftmaxCrossEntropyGradientReduced, const NDArray&, const NDArray&, const NDArray&, double,
                    NDArray&, const Stream&);

} // namespace impl
} // namespace hetu
