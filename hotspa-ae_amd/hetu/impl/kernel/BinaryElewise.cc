// AddElewiseCuda / SubElewiseCuda / MulElewiseCuda / DivElewiseCuda: arguments
// and meaning of hetu/impl/kernel/BinaryElewise.cu of the reference.  Operands
// broadcast to the output's shape (trailing dimensions aligned, extent 1
// repeats) and may have any strides; the output is dense.
#include "hetu/graph/ops/kernel_links.h"
#include "hetu/impl/kernel/kernel_utils.h"
#include "hetu/impl/utils/cpu_utils.h"
#include "hetu/impl/utils/dispatch.h"

namespace hetu {
namespace impl {

namespace {

// element strides of `a` seen through the output's shape: 0 where `a` repeats
std::vector<int64_t> BroadcastStrides(const NDArray& a, const HTShape& out_shape) {
  const int64_t nd = int64_t(out_shape.size()), na = int64_t(a->ndim());
  HT_ASSERT(na <= nd) << "Operand " << a->shape() << " has more dimensions than the output " << out_shape;
  std::vector<int64_t> s(nd, 0);
  for (int64_t i = 0; i < na; ++i) {
    const int64_t o = nd - na + i;
    const int64_t extent = a->shape(i);
    HT_ASSERT(extent == out_shape[o] || extent == 1)
      << "Operand " << a->shape() << " cannot be broadcast to " << out_shape;
    s[o] = (extent == 1 && out_shape[o] != 1) ? 0 : a->stride(i);
  }
  return s;
}

void BinaryElewise(int op, const NDArray& inputA, const NDArray& inputB, NDArray& output, const Stream& stream) {
  HT_ASSERT_CUDA_DEVICE(inputA);
  HT_ASSERT_SAME_DEVICE(inputA, output);
  HT_ASSERT_SAME_DEVICE(inputB, output);
  HT_ASSERT_SAME_DTYPE(inputA, output);
  HT_ASSERT_SAME_DTYPE(inputB, output);
  HT_ASSERT_CONTIGUOUS(output);
  HT_ASSERT(output->ndim() <= 8) << "At most 8 dimensions, got " << output->shape();
  const HTShape expect = NDArrayMeta::Broadcast(inputA->shape(), inputB->shape());
  HT_ASSERT(!expect.empty() || (inputA->ndim() == 0 && inputB->ndim() == 0))
    << "Shapes cannot be broadcast together: " << inputA->shape() << " vs. " << inputB->shape();
  HT_ASSERT(expect == output->shape())
    << "Output " << output->shape() << " does not have the broadcast shape " << expect;
  if (output->numel() == 0) return;

  HIPStream hip_stream(stream);
  hip::DeviceGuard guard(hip_stream.device_id());
  const std::vector<int64_t> sa = BroadcastStrides(inputA, output->shape());
  const std::vector<int64_t> sb = BroadcastStrides(inputB, output->shape());
  std::vector<int64_t> shape(output->shape().begin(), output->shape().end());
  HK_CALL(hk_binary(op, int(output->dtype()), inputA->raw_data_ptr(), inputB->raw_data_ptr(), output->raw_data_ptr(),
                    int(shape.size()), shape.data(), sa.data(), sb.data(), hip_stream));
  NDArray::MarkUsedBy({inputA, inputB, output}, stream);
}

} // namespace

void AddElewiseCuda(const NDArray& inputA, const NDArray& inputB, NDArray& output, const Stream& stream) {
  BinaryElewise(HK_BINARY_ADD, inputA, inputB, output, stream);
}
void SubElewiseCuda(const NDArray& inputA, const NDArray& inputB, NDArray& output, const Stream& stream) {
  BinaryElewise(HK_BINARY_SUB, inputA, inputB, output, stream);
}
void MulElewiseCuda(const NDArray& inputA, const NDArray& inputB, NDArray& output, const Stream& stream) {
  BinaryElewise(HK_BINARY_MUL, inputA, inputB, output, stream);
}
void DivElewiseCuda(const NDArray& inputA, const NDArray& inputB, NDArray& output, const Stream& stream) {
  BinaryElewise(HK_BINARY_DIV, inputA, inputB, output, stream);
}

// ---------------------------------------------------------------------------------------------------------
// Host twins (hetu/impl/kernel/BinaryElewise.cc of the reference, oneDNN binary primitives there): the same
// broadcasting, one run along the last dimension at a time.  Floating-point types compute in float (double for
// float64) and round once; the integer types wrap in their own width, a division by zero gives 0 instead of a trap.
// ---------------------------------------------------------------------------------------------------------
namespace {
void BinaryElewiseHost(int op, const char* who, const NDArray& inputA, const NDArray& inputB, NDArray& output,
                       const Stream& stream) {
  HT_ASSERT_CPU_DEVICE(inputA);
  HT_ASSERT_SAME_DEVICE(inputA, output);
  HT_ASSERT_SAME_DEVICE(inputB, output);
  HT_ASSERT_SAME_DTYPE(inputA, output);
  HT_ASSERT_SAME_DTYPE(inputB, output);
  HT_ASSERT_CONTIGUOUS(output);
  HT_ASSERT(output->ndim() <= 8) << "At most 8 dimensions, got " << output->shape();
  const HTShape expect = NDArrayMeta::Broadcast(inputA->shape(), inputB->shape());
  HT_ASSERT(!expect.empty() || (inputA->ndim() == 0 && inputB->ndim() == 0))
    << "Shapes cannot be broadcast together: " << inputA->shape() << " vs. " << inputB->shape();
  HT_ASSERT(expect == output->shape())
    << "Output " << output->shape() << " does not have the broadcast shape " << expect;
  if (output->numel() == 0) return;
  const std::vector<int64_t> sa = BroadcastStrides(inputA, output->shape());
  const std::vector<int64_t> sb = BroadcastStrides(inputB, output->shape());
  const std::vector<int64_t> shape(output->shape().begin(), output->shape().end());
  const int nd = int(shape.size());
  HT_DISPATCH_INTEGER_AND_FLOATING_TYPES(output->dtype(), spec_t, who, [&]() {
    cpu::on_stream(stream, who, [=]() {   // the stride vectors travel with the task
      const spec_t* pa = inputA->data_ptr<spec_t>();
      const spec_t* pb = inputB->data_ptr<spec_t>();
      spec_t* po = output->data_ptr<spec_t>();
      const int64_t n = nd ? shape[size_t(nd - 1)] : 1;
      const int64_t ia = nd ? sa[size_t(nd - 1)] : 0, ib = nd ? sb[size_t(nd - 1)] : 0;
      cpu::for_each_run(nd, shape.data(), sa.data(), sb.data(), [&](int64_t o, int64_t oa, int64_t ob) {
        for (int64_t i = 0; i < n; ++i) po[o + i] = cpu::binary_op<spec_t>(op, pa[oa + i * ia], pb[ob + i * ib]);
      });
    });
  });
}
} // namespace

void AddElewiseCpu(const NDArray& inputA, const NDArray& inputB, NDArray& output, const Stream& stream) {
  BinaryElewiseHost(HK_BINARY_ADD, "AddElewiseCpu", inputA, inputB, output, stream);
}
void SubElewiseCpu(const NDArray& inputA, const NDArray& inputB, NDArray& output, const Stream& stream) {
  BinaryElewiseHost(HK_BINARY_SUB, "SubElewiseCpu", inputA, inputB, output, stream);
}
void MulElewiseCpu(const NDArray& inputA, const NDArray& inputB, NDArray& output, const Stream& stream) {
  BinaryElewiseHost(HK_BINARY_MUL, "MulElewiseCpu", inputA, inputB, output, stream);
}
void DivElewiseCpu(const NDArray& inputA, const NDArray& inputB, NDArray& output, const Stream& stream) {
  BinaryElewiseHost(HK_BINARY_DIV, "DivElewiseCpu", inputA, inputB, output, stream);
}

} // namespace impl
} // namespace hetu
