// SoftmaxCuda / SoftmaxGradientCuda: arguments and meaning of
// hetu/impl/kernel/Softmax.cu:250-310 and :364-404 of the reference.  The array
// is seen as [outer, dim, inner].  The operator takes non-contiguous arrays
// (hetu/graph/ops/Softmax.h:52-54): for a softmax over the last dimension row-pitched
// inputs and outputs go to the kernels as they are; any other input layout is made
// dense first, and a softmax over another dimension needs a dense output.
#include "hetu/graph/ops/kernel_links.h"
#include "hetu/impl/kernel/kernel_utils.h"

namespace hetu {
namespace impl {

namespace {
void SplitAtDim(const NDArray& a, int64_t& dim, int64_t& outer, int64_t& extent, int64_t& inner) {
  dim = NDArrayMeta::ParseAxis(dim, int64_t(a->ndim()));
  outer = inner = 1;
  extent = a->shape(dim);
  for (int64_t i = 0; i < int64_t(a->ndim()); ++i) {
    if (i < dim) outer *= a->shape(i);
    else if (i > dim) inner *= a->shape(i);
  }
}
} // namespace

void SoftmaxCuda(const NDArray& input, NDArray& output, int64_t dim, const Stream& stream) {
  HT_ASSERT_CUDA_DEVICE(input);
  HT_ASSERT_SAME_DEVICE(input, output);
  HT_ASSERT_SAME_SHAPE(input, output);
  HT_ASSERT_SAME_DTYPE(input, output);
  int64_t outer, extent, inner;
  SplitAtDim(input, dim, outer, extent, inner);
  if (input->numel() == 0) return;

  HIPStream hip_stream(stream);
  hip::DeviceGuard guard(hip_stream.device_id());
  if (inner == 1) {
    int64_t x_pitch = extent, y_pitch = extent;
    HT_ASSERT_ROW_PITCHED(output, 1, &y_pitch);
    NDArray x = RowOperand(input, 1, stream, &x_pitch);
    HK_CALL(hk_softmax_fwd_pitched(int(input->dtype()), x->raw_data_ptr(), x_pitch, output->raw_data_ptr(), y_pitch,
                                   outer, extent, hip_stream));
    NDArray::MarkUsedBy({x, output}, stream);
    return;
  }
  HT_ASSERT_CONTIGUOUS(output);
  NDArray x = Dense(input, stream);
  HK_CALL(hk_softmax_fwd(int(input->dtype()), x->raw_data_ptr(), output->raw_data_ptr(), outer, extent, inner,
                         hip_stream));
  NDArray::MarkUsedBy({x, output}, stream);
}

void SoftmaxGradientCuda(const NDArray& input_Y, const NDArray& output_grad, NDArray& input_grad, int64_t dim,
                         const Stream& stream) {
  HT_ASSERT_CUDA_DEVICE(input_Y);
  HT_ASSERT_SAME_DEVICE(input_Y, output_grad);
  HT_ASSERT_SAME_DEVICE(input_Y, input_grad);
  HT_ASSERT_SAME_SHAPE(input_Y, output_grad);
  HT_ASSERT_SAME_SHAPE(input_Y, input_grad);
  HT_ASSERT_SAME_DTYPE(input_Y, output_grad);
  HT_ASSERT_SAME_DTYPE(input_Y, input_grad);
  int64_t outer, extent, inner;
  SplitAtDim(input_Y, dim, outer, extent, inner);
  if (input_Y->numel() == 0) return;

  HIPStream hip_stream(stream);
  hip::DeviceGuard guard(hip_stream.device_id());
  if (inner == 1) {
    int64_t y_pitch = extent, dy_pitch = extent, dx_pitch = extent;
    HT_ASSERT_ROW_PITCHED(input_grad, 1, &dx_pitch);
    NDArray y = RowOperand(input_Y, 1, stream, &y_pitch), dy = RowOperand(output_grad, 1, stream, &dy_pitch);
    HK_CALL(hk_softmax_bwd_pitched(int(input_Y->dtype()), y->raw_data_ptr(), y_pitch, dy->raw_data_ptr(), dy_pitch,
                                   input_grad->raw_data_ptr(), dx_pitch, outer, extent, hip_stream));
    NDArray::MarkUsedBy({y, dy, input_grad}, stream);
    return;
  }
  HT_ASSERT_CONTIGUOUS(input_grad);
  NDArray y = Dense(input_Y, stream), dy = Dense(output_grad, stream);
  HK_CALL(hk_softmax_bwd(int(input_Y->dtype()), y->raw_data_ptr(), dy->raw_data_ptr(), input_grad->raw_data_ptr(),
                         outer, extent, inner, hip_stream));
  NDArray::MarkUsedBy({y, dy, input_grad}, stream);
}

void SoftmaxCpu(const NDArray&, NDArray&, int64_t, const Stream&) {
  HT_NOT_IMPLEMENTED << "Softmax has no host kernel in this build (the reference's is a oneDNN primitive); "
                        "move the arrays to the accelerator";
}

void SoftmaxGradientCpu(const NDArray&, const NDArray&, NDArray&, int64_t, const Stream&) {
  HT_NOT_IMPLEMENTED << "SoftmaxGradient has no host kernel in this build; move the arrays to the accelerator";
}

} // namespace impl
} // namespace hetu
