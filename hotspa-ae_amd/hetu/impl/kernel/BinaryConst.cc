// AddConstCuda / SubConstCuda / MulConstCuda / DivConstCuda: arguments and
// meaning of hetu/impl/kernel/BinaryConst.cu:10-53 of the reference.  The
// constant is the LEFT operand (SubConst is value - x, DivConst value / x) and
// is rounded to the array's type before it is used.
#include "hetu/graph/ops/kernel_links.h"
#include "hetu/impl/kernel/kernel_utils.h"

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

#define HT_NO_CPU_CONST(name)                                                                        \
  void name##Cpu(const NDArray&, double, NDArray&, const Stream&) {                                  \
    HT_NOT_IMPLEMENTED << #name << " has no CPU kernel in this build (the product path is the GPU)"; \
  }
HT_NO_CPU_CONST(AddConst)
HT_NO_CPU_CONST(SubConst)
HT_NO_CPU_CONST(MulConst)
HT_NO_CPU_CONST(DivConst)
#undef HT_NO_CPU_CONST

} // namespace impl
} // namespace hetu
