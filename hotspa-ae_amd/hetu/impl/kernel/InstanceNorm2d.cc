// InstanceNormCuda / InstanceNormGradientCuda: arguments and meaning of
// hetu/impl/kernel/InstanceNorm2d.cu:60-103 and :191-290 of the reference.  An
// instance norm of [N, C, H, W] is a layer norm without scale and bias over the
// H*W elements of each of the N*C planes, so both run on the layer-norm kernels
// (statistics are mean and variance in the data dtype, one per plane).
#include "hetu/graph/ops/kernel_links.h"
#include "hetu/impl/kernel/kernel_utils.h"

namespace hetu {
namespace impl {

namespace {
void Planes(const NDArray& in_arr, int64_t& rows, int64_t& cols) {
  HT_ASSERT(in_arr->ndim() == 4) << "instance norm expects [N, C, H, W], got " << in_arr->shape();
  rows = in_arr->shape(0) * in_arr->shape(1);
  cols = in_arr->shape(2) * in_arr->shape(3);
}
} // namespace

void InstanceNormCuda(const NDArray& in_arr, NDArray& mean_arr, NDArray& var_arr, NDArray& out_arr, float eps,
                      const Stream& stream) {
  HT_ASSERT_CUDA_DEVICE(in_arr);
  HT_ASSERT_SAME_DEVICE(in_arr, mean_arr);
  HT_ASSERT_SAME_DEVICE(in_arr, var_arr);
  HT_ASSERT_SAME_DEVICE(in_arr, out_arr);
  HT_ASSERT_SAME_SHAPE(in_arr, out_arr);
  HT_ASSERT_SAME_DTYPE(in_arr, out_arr);
  HT_ASSERT_SAME_DTYPE(in_arr, mean_arr);
  HT_ASSERT_SAME_DTYPE(in_arr, var_arr);
  HT_ASSERT_CONTIGUOUS(out_arr);
  HT_ASSERT_CONTIGUOUS(mean_arr);
  HT_ASSERT_CONTIGUOUS(var_arr);
  int64_t rows, cols;
  Planes(in_arr, rows, cols);
  HT_ASSERT(int64_t(mean_arr->numel()) == rows && int64_t(var_arr->numel()) == rows)
    << "statistics must hold one value per plane (" << rows << ")";
  if (in_arr->numel() == 0) return;

  HIPStream hip_stream(stream);
  hip::DeviceGuard guard(hip_stream.device_id());
  NDArray x = Dense(in_arr, stream);
  const int dt = int(in_arr->dtype());
  HK_CALL(hk_layer_norm_fwd(dt, x->raw_data_ptr(), /*gamma=*/nullptr, /*beta=*/nullptr, out_arr->raw_data_ptr(),
                            mean_arr->raw_data_ptr(), var_arr->raw_data_ptr(), dt, HK_STAT_VAR, rows, cols, eps,
                            hip_stream));
  NDArray::MarkUsedBy({x, mean_arr, var_arr, out_arr}, stream);
}

void InstanceNormGradientCuda(const NDArray& out_grads, const NDArray& in_arr, NDArray& grad_arr,
                              const NDArray& mean_arr, const NDArray& var_arr, float eps, const Stream& stream) {
  HT_ASSERT_CUDA_DEVICE(out_grads);
  HT_ASSERT_SAME_DEVICE(out_grads, in_arr);
  HT_ASSERT_SAME_DEVICE(out_grads, grad_arr);
  HT_ASSERT_SAME_DEVICE(out_grads, mean_arr);
  HT_ASSERT_SAME_DEVICE(out_grads, var_arr);
  HT_ASSERT_SAME_SHAPE(out_grads, in_arr);
  HT_ASSERT_SAME_SHAPE(out_grads, grad_arr);
  HT_ASSERT_SAME_DTYPE(out_grads, in_arr);
  HT_ASSERT_SAME_DTYPE(out_grads, grad_arr);
  HT_ASSERT_SAME_DTYPE(out_grads, mean_arr);
  HT_ASSERT_SAME_DTYPE(out_grads, var_arr);
  HT_ASSERT_CONTIGUOUS(grad_arr);
  int64_t rows, cols;
  Planes(in_arr, rows, cols);
  HT_ASSERT(int64_t(mean_arr->numel()) == rows && int64_t(var_arr->numel()) == rows)
    << "statistics must hold one value per plane (" << rows << ")";
  if (in_arr->numel() == 0) return;

  HIPStream hip_stream(stream);
  hip::DeviceGuard guard(hip_stream.device_id());
  NDArray dy = Dense(out_grads, stream), x = Dense(in_arr, stream);
  NDArray mean = Dense(mean_arr, stream), var = Dense(var_arr, stream);
  const int dt = int(in_arr->dtype());
  // no scale, no bias: nothing to sum over the planes, so no workspace either
  HK_CALL(hk_layer_norm_bwd(dt, dy->raw_data_ptr(), x->raw_data_ptr(), /*gamma=*/nullptr, /*beta=*/nullptr,
                            mean->raw_data_ptr(), var->raw_data_ptr(), dt, HK_STAT_VAR, grad_arr->raw_data_ptr(),
                            /*dgamma=*/nullptr, /*dbeta=*/nullptr, rows, cols, eps, /*memory_efficient=*/0,
                            /*clamp_gamma=*/0, /*workspace=*/nullptr, 0, hip_stream));
  NDArray::MarkUsedBy({dy, x, mean, var, grad_arr}, stream);
}

void InstanceNormCpu(const NDArray&, NDArray&, NDArray&, NDArray&, float, const Stream&) {
  HT_NOT_IMPLEMENTED << "InstanceNorm has no host kernel in this build; move the arrays to the accelerator";
}

void InstanceNormGradientCpu(const NDArray&, const NDArray&, NDArray&, const NDArray&, const NDArray&, float,
                             const Stream&) {
  HT_NOT_IMPLEMENTED << "InstanceNormGradient has no host kernel in this build; move the arrays to the accelerator";
}

} // namespace impl
} // namespace hetu
