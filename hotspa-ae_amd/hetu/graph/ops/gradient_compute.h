// What the gradient operators of the reductions and of the reduced losses compute, as plain functions over
// NDArrays: the DoCompute bodies of ReduceGradientOpImpl (hetu/graph/ops/Reduce.cc:153-165, with the constant
// of MakeReduceGradientOp, :246-265), SCESGradOpImpl (hetu/graph/ops/SoftmaxCrossEntropySparse.cc:64-85) and
// SCEGradOpImpl (hetu/graph/ops/SoftmaxCrossEntropy.cc:59-80) of the reference, without the graph around them.
#pragma once

#include <vector>

#include "hetu/core/ndarray.h"
#include "hetu/core/reduction_type.h"

namespace hetu {
namespace graph {

using HTKeepDims = std::vector<bool>;

// Gradient of reduce(input, reduction, axes, keepdims) with respect to input: grad_output laid back over
// input_shape, times 1 / (product of the reduced extents) for kMEAN.  kSUM and kMEAN only.  keepdims holds one
// flag per axis or a single flag for all.
NDArray ReduceGradientCompute(const NDArray& grad_output, const HTShape& input_shape, ReductionType reduction,
                              const HTAxes& axes, const HTKeepDims& keepdims, StreamIndex stream_id,
                              NDArray& output);

// Gradient of NDArray::sceloss(preds, labels, ignored_index, reduction) with respect to preds.  grad_output is
// one value for kMEAN / kSUM, one value per row for kNONE.  `fused` false runs the reference's two steps
// (broadcast the value times 1/rows into a [rows] array, then the gradient kernel); true hands the value and
// the factor to the gradient kernel, which needs no array in between; both give the same bits.
NDArray SCESGradCompute(const NDArray& preds, const NDArray& labels, const NDArray& grad_output,
                        int64_t ignored_index, ReductionType reduction, StreamIndex stream_id, NDArray& output,
                        bool fused = true);

// The same for dense labels of the predictions' shape (NDArray::sceloss without ignored_index).
NDArray SCEGradCompute(const NDArray& preds, const NDArray& labels, const NDArray& grad_output,
                       ReductionType reduction, StreamIndex stream_id, NDArray& output, bool fused = true);

} // namespace graph
} // namespace hetu
