#include "hetu/graph/ops/gradient_compute.h"

#include "hetu/graph/ops/kernel_links.h"
#include "hetu/impl/utils/dispatch.h"

namespace hetu {
namespace graph {

namespace {
NDArray OutputOrNew(NDArray& output, const HTShape& shape, const NDArray& like, StreamIndex stream_id) {
  if (output.is_defined()) {
    HT_ASSERT(output->shape() == shape) << "output has shape " << output->shape() << ", expected " << shape;
    return output;
  }
  return NDArray::empty(shape, like->device(), like->dtype(), stream_id);
}

HTShape RowsShape(const NDArray& preds) {
  HT_ASSERT(preds->ndim() >= 1) << "predictions need at least one dimension";
  HTShape rows_shape(preds->shape().begin(), preds->shape().end() - 1);
  if (rows_shape.empty()) rows_shape = {1};
  return rows_shape;
}

// 1 / rows as the reference forms it: in single precision (`1.0f / broadcasted->numel()`)
double MeanFactor(const HTShape& rows_shape) {
  size_t rows = 1;
  for (int64_t extent : rows_shape) rows *= size_t(extent);
  return double(1.0f / float(rows));
}

// the [rows] array of per-row gradients the reference's two-step form builds
NDArray BroadcastLossGradient(const NDArray& preds, const NDArray& grad_output, ReductionType reduction,
                              StreamIndex stream_id) {
  const HTShape rows_shape = RowsShape(preds);
  NDArray broadcasted = NDArray::empty(rows_shape, preds->device(), preds->dtype(), stream_id);
  Stream stream(preds->device(), stream_id);
  if (reduction == kMEAN) {
    HT_DISPATCH_KERNEL_CPU_AND_CUDA(preds->device().type(), "LossGradient", hetu::impl::BroadcastShapeMul,
                                    grad_output, MeanFactor(rows_shape), broadcasted, HTAxes(), stream);
  } else {
    HT_DISPATCH_KERNEL_CPU_AND_CUDA(preds->device().type(), "LossGradient", hetu::impl::BroadcastShape, grad_output,
                                    broadcasted, HTAxes(), stream);
  }
  return broadcasted;
}

void CheckReduction(ReductionType reduction) {
  HT_ASSERT(reduction == kSUM || reduction == kMEAN || reduction == kNONE)
    << "Unsupported reduction type '" << reduction << "' for loss operators. Expected: ['mean', 'sum', 'none']";
}
} // namespace

NDArray ReduceGradientCompute(const NDArray& grad_output, const HTShape& input_shape, ReductionType reduction,
                              const HTAxes& axes, const HTKeepDims& keepdims, StreamIndex stream_id,
                              NDArray& output) {
  HT_ASSERT(reduction == kSUM || reduction == kMEAN)
    << "ReduceGradient: only the sum and the mean lay their output's gradient back over the input unchanged, got '"
    << reduction << "'";
  const int64_t ndim = int64_t(input_shape.size());
  HTAxes parsed = axes;
  if (parsed.empty())
    for (int64_t i = 0; i < ndim; ++i) parsed.push_back(i);
  parsed = NDArrayMeta::ParseAxes(parsed, ndim);
  HT_ASSERT(keepdims.size() == parsed.size() || keepdims.size() == 1)
    << "ReduceGradient: " << keepdims.size() << " keepdims flags for " << parsed.size() << " axes";
  HTAxes add_axes;
  int64_t mean_multiplier = 1;
  for (size_t i = 0; i < parsed.size(); ++i) {
    mean_multiplier *= input_shape[size_t(parsed[i])];
    if (!(keepdims.size() == 1 ? keepdims[0] : keepdims[i])) add_axes.push_back(parsed[i]);
  }
  NDArray out = OutputOrNew(output, input_shape, grad_output, stream_id);
  Stream stream(grad_output->device(), stream_id);
  // a gradient of fewer dimensions than the input names the dropped ones; when every axis was dropped the
  // reduction's output is [1], which right-aligns by itself
  const bool name_axes = !add_axes.empty() && int64_t(grad_output->ndim()) + int64_t(add_axes.size()) == ndim;
  const HTShape axes_arg = name_axes ? add_axes : HTShape();
  if (reduction == kMEAN) {
    HT_DISPATCH_KERNEL_CPU_AND_CUDA(grad_output->device().type(), "ReduceGradient", hetu::impl::BroadcastShapeMul,
                                    grad_output, 1.0 / double(mean_multiplier), out, axes_arg, stream);
  } else {
    HT_DISPATCH_KERNEL_CPU_AND_CUDA(grad_output->device().type(), "ReduceGradient", hetu::impl::BroadcastShape,
                                    grad_output, out, axes_arg, stream);
  }
  return out;
}

NDArray SCESGradCompute(const NDArray& preds, const NDArray& labels, const NDArray& grad_output,
                        int64_t ignored_index, ReductionType reduction, StreamIndex stream_id, NDArray& output,
                        bool fused) {
  CheckReduction(reduction);
  NDArray out = OutputOrNew(output, preds->shape(), preds, stream_id);
  Stream stream(preds->device(), stream_id);
  if (reduction == kNONE) {
    HT_DISPATCH_KERNEL_CPU_AND_CUDA(preds->device().type(), "SCESGrad", hetu::impl::SoftmaxCrossEntropySparseGradient,
                                    preds, labels, grad_output, out, ignored_index, stream);
  } else if (fused) {
    HT_ASSERT(preds->device().is_cuda()) << "the fused loss gradient runs on the GPU only";
    const double factor = reduction == kMEAN ? MeanFactor(RowsShape(preds)) : 1.0;
    hetu::impl::SoftmaxCrossEntropySparseGradientReducedCuda(preds, labels, grad_output, factor, out, ignored_index,
                                                             stream);
  } else {
    NDArray broadcasted = BroadcastLossGradient(preds, grad_output, reduction, stream_id);
    HT_DISPATCH_KERNEL_CPU_AND_CUDA(preds->device().type(), "SCESGrad", hetu::impl::SoftmaxCrossEntropySparseGradient,
                                    preds, labels, broadcasted, out, ignored_index, stream);
  }
  return out;
}

NDArray SCEGradCompute(const NDArray& preds, const NDArray& labels, const NDArray& grad_output,
                       ReductionType reduction, StreamIndex stream_id, NDArray& output, bool fused) {
  CheckReduction(reduction);
  NDArray out = OutputOrNew(output, preds->shape(), preds, stream_id);
  Stream stream(preds->device(), stream_id);
  if (reduction == kNONE) {
    HT_DISPATCH_KERNEL_CPU_AND_CUDA(preds->device().type(), "SCEGrad", hetu::impl::SoftmaxCrossEntropyGradient, preds,
                                    labels, grad_output, out, stream);
  } else if (fused) {
    HT_ASSERT(preds->device().is_cuda()) << "the fused loss gradient runs on the GPU only";
    const double factor = reduction == kMEAN ? MeanFactor(RowsShape(preds)) : 1.0;
    hetu::impl::SoftmaxCrossEntropyGradientReducedCuda(preds, labels, grad_output, factor, out, stream);
  } else {
    NDArray broadcasted = BroadcastLossGradient(preds, grad_output, reduction, stream_id);
    HT_DISPATCH_KERNEL_CPU_AND_CUDA(preds->device().type(), "SCEGrad", hetu::impl::SoftmaxCrossEntropyGradient, preds,
                                    labels, broadcasted, out, stream);
  }
  return out;
}

} // namespace graph
} // namespace hetu
