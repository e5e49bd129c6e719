// BroadcastShapeCuda / BroadcastShapeMulCuda: arguments and meaning of
// hetu/impl/kernel/BroadcastShape.cu:30-99 and :119-186 of the reference.
//
// The input's dimensions are laid over the output's: with no add_axes they are
// right-aligned (leading output dimensions broadcast); with add_axes the first
// (output ndim - input ndim) of them name output dimensions the input lacks and
// the input's own dimensions fill the remaining positions in order.  An input
// extent of 1 broadcasts.  The reference trusts that every other input extent
// equals the output's (a mismatch reads out of place there); here it is checked.
#include "hetu/graph/ops/kernel_links.h"
#include "hetu/impl/kernel/kernel_utils.h"
#include "hetu/impl/utils/cpu_utils.h"
#include "hetu/impl/utils/dispatch.h"

namespace hetu {
namespace impl {

namespace {
// The input's strides per output dimension (0 where it broadcasts), checked; false when there is nothing to do.
bool BroadcastLayout(const char* who, const NDArray& input, const NDArray& output, const HTShape& add_axes,
                     int64_t out_shape[8], int64_t in_strides[8]) {
  HT_ASSERT_SAME_DEVICE(input, output);
  HT_ASSERT_SAME_DTYPE(input, output);
  HT_ASSERT_CONTIGUOUS(output);
  if (output->numel() == 0 || input->numel() == 0) return false;

  const int in_nd = int(input->ndim()), out_nd = int(output->ndim());
  HT_ASSERT(in_nd <= out_nd) << who << ": input " << input->shape() << " has more dimensions than output "
                             << output->shape();
  HT_ASSERT(out_nd <= 8) << who << ": at most 8 dimensions, got " << out_nd;
  const int diff = out_nd - in_nd;
  // which input dimension sits at each output position (-1: none, the position is broadcast)
  std::vector<int> source(size_t(out_nd), -1);
  if (add_axes.empty()) {
    for (int i = diff; i < out_nd; ++i) source[size_t(i)] = i - diff;
  } else {
    HT_ASSERT(int(add_axes.size()) >= diff)
      << who << ": " << diff << " dimensions to add but only " << add_axes.size() << " axes named";
    std::vector<bool> added(size_t(out_nd), false);
    for (int i = 0; i < diff; ++i) {
      HT_ASSERT(add_axes[size_t(i)] >= 0 && add_axes[size_t(i)] < out_nd)
        << who << ": axis " << add_axes[size_t(i)] << " outside the output's " << out_nd << " dimensions";
      HT_ASSERT(!added[size_t(add_axes[size_t(i)])]) << who << ": axis " << add_axes[size_t(i)] << " named twice";
      added[size_t(add_axes[size_t(i)])] = true;
    }
    int next = 0;
    for (int i = 0; i < out_nd; ++i)
      if (!added[size_t(i)]) source[size_t(i)] = next++;
  }
  for (int i = 0; i < out_nd; ++i) {
    out_shape[i] = output->shape(i);
    in_strides[i] = 0;
    const int src = source[size_t(i)];
    if (src < 0) continue;
    const int64_t extent = input->shape(src);
    HT_ASSERT(extent == 1 || extent == out_shape[i])
      << who << ": input " << input->shape() << " does not broadcast to " << output->shape() << " (add_axes "
      << add_axes << "): extent " << extent << " meets " << out_shape[i] << " at output dimension " << i;
    if (extent > 1) in_strides[i] = input->stride(src);
  }
  return true;
}

void Broadcast(const char* who, const NDArray& input, bool multiply, double const_value, NDArray& output,
               const HTShape& add_axes, const Stream& stream) {
  HT_ASSERT_CUDA_DEVICE(input);
  int64_t out_shape[8], in_strides[8];
  if (!BroadcastLayout(who, input, output, add_axes, out_shape, in_strides)) return;
  const int out_nd = int(output->ndim());
  HIPStream hip_stream(stream);
  hip::DeviceGuard guard(hip_stream.device_id());
  HK_CALL(hk_broadcast(int(input->dtype()), input->raw_data_ptr(), multiply ? 1 : 0, const_value,
                       output->raw_data_ptr(), out_nd, out_shape, in_strides, hip_stream));
  NDArray::MarkUsedBy({input, output}, stream);
}
} // namespace

void BroadcastShapeCuda(const NDArray& input, NDArray& output, const HTShape& add_axes, const Stream& stream) {
  Broadcast("BroadcastShape", input, false, 1.0, output, add_axes, stream);
}

void BroadcastShapeMulCuda(const NDArray& input, double const_value, NDArray& output, const HTShape& add_axes,
                           const Stream& stream) {
  Broadcast("BroadcastShapeMul", input, true, const_value, output, add_axes, stream);
}

// Host twins (hetu/impl/kernel/BroadcastShape.cc of the reference): the same layout, copied (or multiplied by
// the constant rounded to the array's type) one run along the last dimension at a time.
namespace {
void BroadcastHost(const char* who, const NDArray& input, bool multiply, double const_value, NDArray& output,
                   const HTShape& add_axes, const Stream& stream) {
  HT_ASSERT_CPU_DEVICE(input);
  int64_t out_shape[8], in_strides[8], none[8] = {0, 0, 0, 0, 0, 0, 0, 0};
  if (!BroadcastLayout(who, input, output, add_axes, out_shape, in_strides)) return;
  const int nd = int(output->ndim());
  HT_DISPATCH_INTEGER_AND_FLOATING_TYPES(output->dtype(), spec_t, who, [&]() {
    cpu::on_stream(stream, who, [=]() {   // the layout arrays are copied into the task
      const spec_t* pi = input->data_ptr<spec_t>();
      spec_t* po = output->data_ptr<spec_t>();
      const spec_t c = static_cast<spec_t>(const_value);
      const int64_t n = nd ? out_shape[nd - 1] : 1, step = nd ? in_strides[nd - 1] : 0;
      cpu::for_each_run(nd, out_shape, in_strides, none, [&](int64_t o, int64_t oi, int64_t) {
        if (multiply) {
          for (int64_t i = 0; i < n; ++i) po[o + i] = cpu::binary_op<spec_t>(2, pi[oi + i * step], c);
        } else {
          for (int64_t i = 0; i < n; ++i) po[o + i] = pi[oi + i * step];
        }
      });
    });
  });
}
} // namespace

void BroadcastShapeCpu(const NDArray& input, NDArray& output, const HTShape& add_axes, const Stream& stream) {
  BroadcastHost("BroadcastShape", input, false, 1.0, output, add_axes, stream);
}
void BroadcastShapeMulCpu(const NDArray& input, double const_value, NDArray& output, const HTShape& add_axes,
                          const Stream& stream) {
  BroadcastHost("BroadcastShapeMul", input, true, const_value, output, add_axes, stream);
}

} // namespace impl
} // namespace hetu
