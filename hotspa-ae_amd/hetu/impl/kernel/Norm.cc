// NormCuda / NormGradientCuda: arguments and meaning of
// hetu/impl/kernel/Norm1.cu:99-133 and :135-186 of the reference: the p-norm of
// one dimension, (sum |x|^p)^(1/p), and its gradient.  A negative dim counts
// from the end.
#include "hetu/graph/ops/kernel_links.h"
#include "hetu/impl/kernel/kernel_utils.h"

namespace hetu {
namespace impl {

void NormCuda(const NDArray& input, NDArray& output, int64_t dim, int64_t p, const Stream& stream) {
  HT_ASSERT_CUDA_DEVICE(input);
  HT_ASSERT_SAME_DEVICE(input, output);
  HT_ASSERT_SAME_DTYPE(input, output);
  HT_ASSERT_CONTIGUOUS(output);
  HT_VALUE_ERROR_IF(p < 1) << "The norm's exponent must be at least 1, got " << p;
  const int64_t nd = int64_t(input->ndim());
  HT_NOT_IMPLEMENTED_IF(nd > 8) << "norms of arrays with more than 8 dimensions";
  dim = NDArrayMeta::ParseAxis(dim, nd);
  size_t kept = 1;
  for (int64_t i = 0; i < nd; ++i)
    if (i != dim) kept *= size_t(input->shape(i));
  HT_ASSERT(output->numel() == kept) << "output " << output->shape() << " does not hold the " << kept
                                     << " norms of " << input->shape() << " over dimension " << dim;
  if (kept == 0) return;

  HIPStream hip_stream(stream);
  hip::DeviceGuard guard(hip_stream.device_id());
  size_t ws_bytes = 0;
  HK_CALL(hk_reduce_workspace_bytes(int(input->dtype()), int(nd), input->shape().data(), input->stride().data(), 1,
                                    &dim, &ws_bytes));
  NDArray ws = Scratch(ws_bytes, input->device(), stream);
  HK_CALL(hk_norm(int(input->dtype()), input->raw_data_ptr(), output->raw_data_ptr(), int(nd), input->shape().data(),
                  input->stride().data(), dim, p, MutPtrOrNull(ws), ws_bytes, hip_stream));
  NDArray::MarkUsedBy({input, output, ws}, stream);
}

void NormGradientCuda(const NDArray& input, const NDArray& output, const NDArray& output_grad, NDArray& input_grad,
                      int64_t dim, int64_t p, const Stream& stream) {
  HT_ASSERT_CUDA_DEVICE(input);
  HT_ASSERT_SAME_DEVICE(input, output);
  HT_ASSERT_SAME_DEVICE(input, output_grad);
  HT_ASSERT_SAME_DEVICE(input, input_grad);
  HT_ASSERT_SAME_SHAPE(input, input_grad);
  HT_ASSERT_SAME_DTYPE(input, output);
  HT_ASSERT_SAME_DTYPE(input, output_grad);
  HT_ASSERT_SAME_DTYPE(input, input_grad);
  HT_ASSERT_CONTIGUOUS(input_grad);
  HT_VALUE_ERROR_IF(p < 1) << "The norm's exponent must be at least 1, got " << p;
  const int64_t nd = int64_t(input->ndim());
  dim = NDArrayMeta::ParseAxis(dim, nd);
  int64_t before = 1, after = 1;
  for (int64_t i = 0; i < nd; ++i) {
    if (i < dim) before *= input->shape(i);
    else if (i > dim) after *= input->shape(i);
  }
  const int64_t reduce_size = input->shape(dim);
  HT_ASSERT(int64_t(output->numel()) == before * after && int64_t(output_grad->numel()) == before * after)
    << "norm " << output->shape() << " and its gradient " << output_grad->shape() << " must hold " << before * after
    << " values for " << input->shape() << " over dimension " << dim;
  if (input->numel() == 0) return;

  HIPStream hip_stream(stream);
  hip::DeviceGuard guard(hip_stream.device_id());
  NDArray x = Dense(input, stream), n = Dense(output, stream), g = Dense(output_grad, stream);
  HK_CALL(hk_norm_bwd(int(input->dtype()), x->raw_data_ptr(), n->raw_data_ptr(), g->raw_data_ptr(),
                      input_grad->raw_data_ptr(), before, reduce_size, after, p, hip_stream));
  NDArray::MarkUsedBy({x, n, g, input_grad}, stream);
}

void NormCpu(const NDArray&, NDArray&, int64_t, int64_t, const Stream&) {
  HT_NOT_IMPLEMENTED << "Norm has no CPU kernel in this build (the product path is the GPU)";
}
void NormGradientCpu(const NDArray&, const NDArray&, const NDArray&, NDArray&, int64_t, int64_t, const Stream&) {
  HT_NOT_IMPLEMENTED << "NormGradient has no CPU kernel in this build (the product path is the GPU)";
}

} // namespace impl
} // namespace hetu
