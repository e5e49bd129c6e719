// ExpCuda, LogCuda, OppositeCuda, SqrtCuda: arguments and meaning of
// hetu/impl/kernel/Exp.cu:12-29, Log.cu, Opposite.cu and Sqrt.cu of the
// reference (one launch_loop_kernel each there, one hk_unary call here).
#include "hetu/graph/ops/kernel_links.h"
#include "hetu/impl/kernel/kernel_utils.h"

namespace hetu {
namespace impl {

namespace {
void Unary(int op, const NDArray& input, NDArray& output, const Stream& stream) {
  HT_ASSERT_CUDA_DEVICE(input);
  HT_ASSERT_SAME_DEVICE(input, output);
  HT_ASSERT_SAME_SHAPE(input, output);
  HT_ASSERT_SAME_DTYPE(input, output);
  HT_ASSERT_CONTIGUOUS(output);
  if (input->numel() == 0) return;
  HIPStream hip_stream(stream);
  hip::DeviceGuard guard(hip_stream.device_id());
  NDArray x = Dense(input, stream);
  HK_CALL(hk_unary(op, int(input->dtype()), x->raw_data_ptr(), output->raw_data_ptr(), int64_t(input->numel()),
                   hip_stream));
  NDArray::MarkUsedBy({x, output}, stream);
}
} // namespace

void ExpCuda(const NDArray& input, NDArray& output, const Stream& stream) { Unary(HK_UNARY_EXP, input, output, stream); }
void LogCuda(const NDArray& input, NDArray& output, const Stream& stream) { Unary(HK_UNARY_LOG, input, output, stream); }
void OppositeCuda(const NDArray& input, NDArray& output, const Stream& stream) {
  Unary(HK_UNARY_NEG, input, output, stream);
}
void SqrtCuda(const NDArray& input, NDArray& output, const Stream& stream) { Unary(HK_UNARY_SQRT, input, output, stream); }

#define HT_NO_CPU_UNARY(name)                                                                        \
  void name##Cpu(const NDArray&, NDArray&, const Stream&) {                                          \
    HT_NOT_IMPLEMENTED << #name << " has no CPU kernel in this build (the product path is the GPU)"; \
  }
HT_NO_CPU_UNARY(Exp)
HT_NO_CPU_UNARY(Log)
HT_NO_CPU_UNARY(Opposite)
HT_NO_CPU_UNARY(Sqrt)
#undef HT_NO_CPU_UNARY

} // namespace impl
} // namespace hetu
