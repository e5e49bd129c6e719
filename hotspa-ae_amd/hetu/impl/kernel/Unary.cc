// ExpCuda, LogCuda, OppositeCuda, SqrtCuda: arguments and meaning of
// hetu/impl/kernel/Exp.cu:12-29, Log.cu, Opposite.cu and Sqrt.cu of the
// reference (one launch_loop_kernel each there, one hk_unary call here).
#include "hetu/graph/ops/kernel_links.h"
#include "hetu/impl/kernel/kernel_utils.h"
#include "hetu/impl/utils/cpu_utils.h"
#include "hetu/impl/utils/dispatch.h"

#include <cmath>

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

// Host twins (hetu/impl/kernel/Exp.cc, Log.cc, Opposite.cc, Sqrt.cc of the reference): one pass, float arithmetic
// (double for float64) rounded once; the negation also takes the integer types and wraps.
namespace {
void UnaryHost(int op, const char* who, const NDArray& input, NDArray& output, const Stream& stream) {
  HT_ASSERT_CPU_DEVICE(input);
  HT_ASSERT_SAME_DEVICE(input, output);
  HT_ASSERT_SAME_SHAPE(input, output);
  HT_ASSERT_SAME_DTYPE(input, output);
  HT_ASSERT_CONTIGUOUS(output);
  if (input->numel() == 0) return;
  const int64_t n = int64_t(input->numel());
  if (op == HK_UNARY_NEG) {
    HT_DISPATCH_INTEGER_AND_FLOATING_TYPES(input->dtype(), spec_t, who, [&]() {
      cpu::on_stream(stream, who, [=]() {
        NDArray x = Dense(input, stream);
        const spec_t* px = x->data_ptr<spec_t>();
        spec_t* po = output->data_ptr<spec_t>();
        cpu::parallel_for(n, [&](int64_t i) { po[i] = cpu::negate<spec_t>(px[i]); });
      });
    });
    return;
  }
  HT_DISPATCH_FLOATING_TYPES(input->dtype(), spec_t, who, [&]() {
    cpu::on_stream(stream, who, [=]() {
      using A = typename cpu::Arith<spec_t>::type;
      NDArray x = Dense(input, stream);
      const spec_t* px = x->data_ptr<spec_t>();
      spec_t* po = output->data_ptr<spec_t>();
      // one loop per operation: the choice stays outside, the exp and sqrt loops vectorise
      if (op == HK_UNARY_EXP) {
        cpu::parallel_for(n, [&](int64_t i) { cpu::st<spec_t, A>(po + i, cpu::exp_(cpu::ld<spec_t, A>(px + i))); });
      } else if (op == HK_UNARY_LOG) {
        cpu::parallel_for(n, [&](int64_t i) { cpu::st<spec_t, A>(po + i, std::log(cpu::ld<spec_t, A>(px + i))); });
      } else {
        cpu::parallel_for(n, [&](int64_t i) { cpu::st<spec_t, A>(po + i, std::sqrt(cpu::ld<spec_t, A>(px + i))); });
      }
    });
  });
}
} // namespace

void ExpCpu(const NDArray& input, NDArray& output, const Stream& stream) { UnaryHost(HK_UNARY_EXP, "ExpCpu", input, output, stream); }
void LogCpu(const NDArray& input, NDArray& output, const Stream& stream) { UnaryHost(HK_UNARY_LOG, "LogCpu", input, output, stream); }
void OppositeCpu(const NDArray& input, NDArray& output, const Stream& stream) {
  UnaryHost(HK_UNARY_NEG, "OppositeCpu", input, output, stream);
}
void SqrtCpu(const NDArray& input, NDArray& output, const Stream& stream) { UnaryHost(HK_UNARY_SQRT, "SqrtCpu", input, output, stream); }

} // namespace impl
} // namespace hetu
