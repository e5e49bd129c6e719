// ReduceCuda / ReduceSumCuda / ReduceMeanCuda / ReduceMaxCuda / ReduceMinCuda /
// ReduceProdCuda: arguments and meaning of hetu/impl/kernel/Reduce.cu:21-59,
// ReduceSum.cu:25-42, ReduceMean.cu:35-55, ReduceMax.cu:28-41, ReduceMin.cu:28-41
// and ReduceProd.cu:26-45 of the reference.  The input may have any strides (the
// kernel plans on shape and strides); the output is written dense.
#include "hetu/graph/ops/kernel_links.h"
#include "hetu/impl/kernel/kernel_utils.h"

namespace hetu {
namespace impl {

namespace {
void LaunchReduce(const NDArray& in_arr, NDArray& out_arr, const int64_t* axes, int64_t num_ax, int op,
                  const Stream& stream) {
  HT_ASSERT_CUDA_DEVICE(in_arr);
  HT_ASSERT_SAME_DEVICE(in_arr, out_arr);
  HT_ASSERT_CONTIGUOUS(out_arr);
  const int64_t nd = int64_t(in_arr->ndim());
  HT_NOT_IMPLEMENTED_IF(nd > 8) << "reductions of arrays with more than 8 dimensions";
  size_t kept = 1;
  std::vector<bool> reduced(nd, false);
  for (int64_t i = 0; i < num_ax; ++i) {
    HT_VALUE_ERROR_IF(axes[i] < 0 || axes[i] >= nd) << "axis " << axes[i] << " out of range for " << in_arr->shape();
    reduced[axes[i]] = true;
  }
  for (int64_t i = 0; i < nd; ++i)
    if (!reduced[i]) kept *= size_t(in_arr->shape(i));
  HT_ASSERT(out_arr->numel() == kept) << "output " << out_arr->shape() << " does not hold the " << kept
                                      << " kept elements of " << in_arr->shape();
  if (kept == 0) return;

  HIPStream hip_stream(stream);
  hip::DeviceGuard guard(hip_stream.device_id());
  size_t ws_bytes = 0;
  HK_CALL(hk_reduce_workspace_bytes(int(in_arr->dtype()), int(nd), in_arr->shape().data(), in_arr->stride().data(),
                                    int(num_ax), axes, &ws_bytes));
  NDArray ws = Scratch(ws_bytes, in_arr->device(), stream);
  HK_CALL(hk_reduce(int(in_arr->dtype()), int(out_arr->dtype()), in_arr->raw_data_ptr(), out_arr->raw_data_ptr(),
                    int(nd), in_arr->shape().data(), in_arr->stride().data(), int(num_ax), axes, op,
                    MutPtrOrNull(ws), ws_bytes, hip_stream));
  NDArray::MarkUsedBy({in_arr, out_arr, ws}, stream);
}
} // namespace

void ReduceSumCuda(const NDArray& in_arr, NDArray& out_arr, const int64_t* axes, int64_t num_ax,
                   const Stream& stream) {
  LaunchReduce(in_arr, out_arr, axes, num_ax, HK_REDUCE_SUM, stream);
}

void ReduceMeanCuda(const NDArray& in_arr, NDArray& out_arr, const int64_t* axes, int64_t num_ax,
                    const Stream& stream) {
  LaunchReduce(in_arr, out_arr, axes, num_ax, HK_REDUCE_MEAN, stream);
}

void ReduceMaxCuda(const NDArray& in_arr, NDArray& out_arr, const int64_t* axes, int64_t num_ax,
                   const Stream& stream) {
  LaunchReduce(in_arr, out_arr, axes, num_ax, HK_REDUCE_MAX, stream);
}

void ReduceMinCuda(const NDArray& in_arr, NDArray& out_arr, const int64_t* axes, int64_t num_ax,
                   const Stream& stream) {
  LaunchReduce(in_arr, out_arr, axes, num_ax, HK_REDUCE_MIN, stream);
}

void ReduceProdCuda(const NDArray& in_arr, NDArray& out_arr, const int64_t* axes, int64_t num_ax,
                    const Stream& stream) {
  LaunchReduce(in_arr, out_arr, axes, num_ax, HK_REDUCE_PROD, stream);
}

void ReduceCuda(const NDArray& input, NDArray& output, const HTAxes& axes, ReductionType red_type,
                const Stream& stream) {
  HT_ASSERT_CUDA_DEVICE(input);
  HT_ASSERT_SAME_DEVICE(input, output);
  HTAxes parsed_axes = NDArrayMeta::ParseAxes(axes, int64_t(input->ndim()));
  switch (red_type) {
    case kSUM: ReduceSumCuda(input, output, parsed_axes.data(), int64_t(parsed_axes.size()), stream); break;
    case kMEAN: ReduceMeanCuda(input, output, parsed_axes.data(), int64_t(parsed_axes.size()), stream); break;
    case kMAX: ReduceMaxCuda(input, output, parsed_axes.data(), int64_t(parsed_axes.size()), stream); break;
    case kMIN: ReduceMinCuda(input, output, parsed_axes.data(), int64_t(parsed_axes.size()), stream); break;
    case kPROD: ReduceProdCuda(input, output, parsed_axes.data(), int64_t(parsed_axes.size()), stream); break;
    case kNONE: HT_NOT_IMPLEMENTED << "Reduction type cannot be none"; break;
    default: HT_VALUE_ERROR << "Unknown reduction type: " << static_cast<int32_t>(red_type);
  }
}

void ReduceCpu(const NDArray&, NDArray&, const HTAxes&, ReductionType, const Stream&) {
  HT_NOT_IMPLEMENTED << "Reduce has no host kernel in this build (the reference's is a oneDNN primitive); move the "
                        "arrays to the accelerator";
}
void ReduceSumCpu(const NDArray&, NDArray&, const int64_t*, int64_t, const Stream&) {
  HT_NOT_IMPLEMENTED << "ReduceSum has no host kernel in this build; move the arrays to the accelerator";
}
void ReduceMeanCpu(const NDArray&, NDArray&, const int64_t*, int64_t, const Stream&) {
  HT_NOT_IMPLEMENTED << "ReduceMean has no host kernel in this build; move the arrays to the accelerator";
}
void ReduceMaxCpu(const NDArray&, NDArray&, const int64_t*, int64_t, const Stream&) {
  HT_NOT_IMPLEMENTED << "ReduceMax has no host kernel in this build; move the arrays to the accelerator";
}
void ReduceMinCpu(const NDArray&, NDArray&, const int64_t*, int64_t, const Stream&) {
  HT_NOT_IMPLEMENTED << "ReduceMin has no host kernel in this build; move the arrays to the accelerator";
}
void ReduceProdCpu(const NDArray&, NDArray&, const int64_t*, int64_t, const Stream&) {
  HT_NOT_IMPLEMENTED << "ReduceProd has no host kernel in this build; move the arrays to the accelerator";
}

} // namespace impl
} // namespace hetu
