// AddConstCuda / SubConstCuda / MulConstCuda / DivConstCuda: arguments and
// meaning of hetu/impl/kernel/BinaryConst.cu:10-53 of the reference.  The
// constant is the LEFT operand (SubConst is value - x, DivConst value / x) and
// is rounded to the array's type before it is used.
#include "hetu/graph/ops/kernel_links.h"
#include "hetu/impl/kernel/kernel_utils.h"
#include "hetu/impl/utils/cpu_utils.h"
#include "hetu/impl/utils/dispatch.h"

namespace hetu {
namespace impl {

namespace {
void BinaryConst(int op, const NDArray& input, double value, NDArray& output, const Stream& stream) {
  HT_ASSERT_CUDA_DEVICE(input);
  HT_ASSERT_SAME_DEVICE(input, output);
  HT_ASSERT_SAME_SHAPE(input, output);
  HT_ASSERT_SAME_DTYPE(input, output);
  HT_ASSERT_CONTIGUOUS(output);
  if (input->numel() == 0) return;
  HIPStream hip_stream(stream);
  hip::DeviceGuard guard(hip_stream.device_id());
  NDArray x = Dense(input, stream);
  HK_CALL(hk_binary_const(op, int(input->dtype()), x->raw_data_ptr(), value, /*scalar_first=*/1,
                          output->raw_data_ptr(), int64_t(input->numel()), hip_stream));
  NDArray::MarkUsedBy({x, output}, stream);
}
} // namespace

void AddConstCuda(const NDArray& input, double value, NDArray& output, const Stream& stream) {
  BinaryConst(HK_BINARY_ADD, input, value, output, stream);
}
void SubConstCuda(const NDArray& input, double value, NDArray& output, const Stream& stream) {
  BinaryConst(HK_BINARY_SUB, input, value, output, stream);
}
void MulConstCuda(const NDArray& input, double value, NDArray& output, const Stream& stream) {
  BinaryConst(HK_BINARY_MUL, input, value, output, stream);
}
void DivConstCuda(const NDArray& input, double value, NDArray& output, const Stream& stream) {
  HT_ASSERT(value != 0) << "Divided by 0.";   // the reference's check (BinaryConst.cu:47)
  BinaryConst(HK_BINARY_DIV, input, value, output, stream);
}

// Host twins (hetu/impl/kernel/BinaryConst.cc of the reference): value op x with the constant rounded to the
// array's type first; arithmetic as in the element-wise twins (float / double, integers wrap, x = 0 under an
// integer division gives 0).
namespace {
void BinaryConstHost(int op, const char* who, const NDArray& input, double value, NDArray& output,
                     const Stream& stream) {
  HT_ASSERT_CPU_DEVICE(input);
  HT_ASSERT_SAME_DEVICE(input, output);
  HT_ASSERT_SAME_SHAPE(input, output);
  HT_ASSERT_SAME_DTYPE(input, output);
  HT_ASSERT_CONTIGUOUS(output);
  if (input->numel() == 0) return;
  const int64_t n = int64_t(input->numel());
  HT_DISPATCH_INTEGER_AND_FLOATING_TYPES(input->dtype(), spec_t, who, [&]() {
    cpu::on_stream(stream, who, [=]() {
      NDArray x = Dense(input, stream);
      const spec_t* px = x->data_ptr<spec_t>();
      spec_t* po = output->data_ptr<spec_t>();
      const spec_t c = static_cast<spec_t>(value);   // the constant in the array's type, as the accelerator path
      cpu::parallel_for(n, [&](int64_t i) { po[i] = cpu::binary_op<spec_t>(op, c, px[i]); });
    });
  });
}
} // namespace

void AddConstCpu(const NDArray& input, double value, NDArray& output, const Stream& stream) {
  BinaryConstHost(HK_BINARY_ADD, "AddConstCpu", input, value, output, stream);
}
void SubConstCpu(const NDArray& input, double value, NDArray& output, const Stream& stream) {
  BinaryConstHost(HK_BINARY_SUB, "SubConstCpu", input, value, output, stream);
}
void MulConstCpu(const NDArray& input, double value, NDArray& output, const Stream& stream) {
  BinaryConstHost(HK_BINARY_MUL, "MulConstCpu", input, value, output, stream);
}
void DivConstCpu(const NDArray& input, double value, NDArray& output, const Stream& stream) {
  HT_ASSERT(value != 0) << "Divided by 0.";
  BinaryConstHost(HK_BINARY_DIV, "DivConstCpu", input, value, output, stream);
}

} // namespace impl
} // namespace hetu
