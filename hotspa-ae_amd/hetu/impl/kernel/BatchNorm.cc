// BatchNormCuda / BatchNormGradientCuda: arguments and meaning of
// hetu/impl/kernel/BatchNorm.cu:8-83 and :84-165 of the reference, which hands the
// work to cuDNN's spatial batch normalisation in training mode.  save_var holds
// what cuDNN saves there: the inverse standard deviation 1 / sqrt(var + eps).
// Scale, bias and every statistic are float32 for float16 / bfloat16 data.
#include "hetu/graph/ops/kernel_links.h"
#include "hetu/impl/kernel/kernel_utils.h"

namespace hetu {
namespace impl {

namespace {
DataType ParamType(DataType data) {
  return (data == kFloat16 || data == kBFloat16) ? kFloat32 : data;
}

void CheckParam(const NDArray& a, DataType dtype, int64_t channels, const char* name) {
  HT_ASSERT(a.is_defined()) << name << " must be given";
  HT_ASSERT(a->is_cuda()) << name << " must live on the GPU";
  HT_ASSERT(a->dtype() == dtype) << name << " must have dtype " << dtype << ", got " << a->dtype();
  HT_ASSERT(int64_t(a->numel()) == channels) << name << " must have one value per channel (" << channels
                                             << "), got " << a->shape();
  HT_ASSERT(a->is_contiguous()) << name << " must be contiguous";
}

void SplitNCHW(const NDArray& x, int64_t& N, int64_t& C, int64_t& HW) {
  HT_ASSERT(x->ndim() >= 2) << "Batch normalisation needs [N, C, ...], got " << x->shape();
  N = x->shape(0);
  C = x->shape(1);
  HW = 1;
  for (size_t i = 2; i < x->ndim(); ++i) HW *= x->shape(int64_t(i));
}
} // namespace

void BatchNormCuda(const NDArray& input_X, const NDArray& bn_scale, const NDArray& bn_bias, NDArray& output_Y,
                   double momentum, double eps, NDArray& running_mean, NDArray& running_var, NDArray& save_mean,
                   NDArray& save_var, const Stream& stream) {
  HT_ASSERT_CUDA_DEVICE(input_X);
  HT_ASSERT_SAME_DEVICE(input_X, bn_scale);
  HT_ASSERT_SAME_DEVICE(input_X, bn_bias);
  HT_ASSERT_SAME_DEVICE(input_X, output_Y);
  HT_ASSERT_SAME_SHAPE(input_X, output_Y);
  HT_ASSERT_SAME_DTYPE(input_X, output_Y);
  HT_ASSERT_CONTIGUOUS(output_Y);
  int64_t N, C, HW;
  SplitNCHW(input_X, N, C, HW);
  const DataType pt = ParamType(input_X->dtype());
  CheckParam(bn_scale, pt, C, "bn_scale");
  CheckParam(bn_bias, pt, C, "bn_bias");
  CheckParam(running_mean, pt, C, "running_mean");
  CheckParam(running_var, pt, C, "running_var");
  CheckParam(save_mean, pt, C, "save_mean");
  CheckParam(save_var, pt, C, "save_var");
  if (input_X->numel() == 0) return;

  HIPStream hip_stream(stream);
  hip::DeviceGuard guard(hip_stream.device_id());
  NDArray x = Dense(input_X, stream);
  size_t ws_bytes = 0;
  HK_CALL(hk_batch_norm_workspace_bytes(int(x->dtype()), N, C, HW, &ws_bytes));
  NDArray ws = Scratch(ws_bytes, x->device(), stream);
  HK_CALL(hk_batch_norm_fwd(int(x->dtype()), x->raw_data_ptr(), bn_scale->raw_data_ptr(), bn_bias->raw_data_ptr(),
                            output_Y->raw_data_ptr(), momentum, eps, running_mean->raw_data_ptr(),
                            running_var->raw_data_ptr(), save_mean->raw_data_ptr(), save_var->raw_data_ptr(), N, C,
                            HW, MutPtrOrNull(ws), ws_bytes, hip_stream));
  NDArray::MarkUsedBy({x, bn_scale, bn_bias, output_Y, running_mean, running_var, save_mean, save_var, ws}, stream);
}

void BatchNormGradientCuda(const NDArray& gradient_Y, const NDArray& input_X, const NDArray& bn_scale,
                           NDArray& gradient_X, NDArray& gradient_bn_scale, NDArray& gradient_bn_bias, double eps,
                           NDArray& save_mean, NDArray& save_var, const Stream& stream) {
  (void) eps;   // already inside the saved inverse standard deviation
  HT_ASSERT_CUDA_DEVICE(gradient_Y);
  HT_ASSERT_SAME_DEVICE(gradient_Y, input_X);
  HT_ASSERT_SAME_DEVICE(gradient_Y, bn_scale);
  HT_ASSERT_SAME_DEVICE(gradient_Y, gradient_X);
  HT_ASSERT_SAME_SHAPE(gradient_Y, input_X);
  HT_ASSERT_SAME_SHAPE(gradient_X, input_X);
  HT_ASSERT_SAME_DTYPE(gradient_Y, input_X);
  HT_ASSERT_SAME_DTYPE(gradient_X, input_X);
  HT_ASSERT_CONTIGUOUS(gradient_X);
  int64_t N, C, HW;
  SplitNCHW(input_X, N, C, HW);
  const DataType pt = ParamType(input_X->dtype());
  CheckParam(bn_scale, pt, C, "bn_scale");
  CheckParam(gradient_bn_scale, pt, C, "gradient_bn_scale");
  CheckParam(gradient_bn_bias, pt, C, "gradient_bn_bias");
  CheckParam(save_mean, pt, C, "save_mean");
  CheckParam(save_var, pt, C, "save_var");
  if (input_X->numel() == 0) return;

  HIPStream hip_stream(stream);
  hip::DeviceGuard guard(hip_stream.device_id());
  NDArray x = Dense(input_X, stream), dy = Dense(gradient_Y, stream);
  size_t ws_bytes = 0;
  HK_CALL(hk_batch_norm_workspace_bytes(int(x->dtype()), N, C, HW, &ws_bytes));
  NDArray ws = Scratch(ws_bytes, x->device(), stream);
  HK_CALL(hk_batch_norm_bwd(int(x->dtype()), dy->raw_data_ptr(), x->raw_data_ptr(), bn_scale->raw_data_ptr(),
                            gradient_X->raw_data_ptr(), gradient_bn_scale->raw_data_ptr(),
                            gradient_bn_bias->raw_data_ptr(), save_mean->raw_data_ptr(), save_var->raw_data_ptr(), N,
                            C, HW, MutPtrOrNull(ws), ws_bytes, hip_stream));
  NDArray::MarkUsedBy({dy, x, bn_scale, gradient_X, gradient_bn_scale, gradient_bn_bias, save_mean, save_var, ws},
                      stream);
}

void BatchNormCpu(const NDArray&, const NDArray&, const NDArray&, NDArray&, double, double, NDArray&, NDArray&,
                  NDArray&, NDArray&, const Stream&) {
  HT_NOT_IMPLEMENTED << "BatchNorm has no CPU kernel in this build (the product path is the GPU)";
}
void BatchNormGradientCpu(const NDArray&, const NDArray&, const NDArray&, NDArray&, NDArray&, NDArray&, double,
                          NDArray&, NDArray&, const Stream&) {
  HT_NOT_IMPLEMENTED << "BatchNormGradient has no CPU kernel in this build (the product path is the GPU)";
}

} // namespace impl
} // namespace hetu
