// NLLLossCuda / NLLLossGradientCuda: arguments and meaning of
// hetu/impl/kernel/NLLLoss.cu:43-86 and :88-128 of the reference.
#include "hetu/graph/ops/kernel_links.h"
#include "hetu/impl/kernel/kernel_utils.h"
#include "hetu/impl/utils/cpu_utils.h"
#include "hetu/impl/utils/dispatch.h"

#include <cmath>
#include <limits>

namespace hetu {
namespace impl {

void NLLLossCuda(const NDArray& pred, const NDArray& label, NDArray& loss, const Stream& stream) {
  HT_ASSERT_CUDA_DEVICE(pred);
  HT_ASSERT_SAME_DEVICE(pred, label);
  HT_ASSERT_SAME_DEVICE(pred, loss);
  HT_ASSERT_SAME_SHAPE(label, loss);
  HT_ASSERT_SAME_DTYPE(pred, loss);
  HT_ASSERT(label->dtype() == kInt64) << "labels must be int64 class ids, got " << label->dtype();
  HT_ASSERT(pred->ndim() == label->ndim() + 1);
  for (size_t i = 0; i < label->ndim(); i++) HT_ASSERT(pred->shape(i) == label->shape(i));
  HT_ASSERT_CONTIGUOUS(loss);
  int64_t rows = 1;
  for (size_t i = 0; i < label->ndim(); i++) rows *= label->shape(i);
  const int64_t cols = pred->shape(pred->ndim() - 1);
  if (rows == 0) return;

  HIPStream hip_stream(stream);
  hip::DeviceGuard guard(hip_stream.device_id());
  NDArray p = Dense(pred, stream), l = Dense(label, stream);
  HK_CALL(hk_nll_loss_fwd(int(pred->dtype()), p->raw_data_ptr(), l->data_ptr<int64_t>(), loss->raw_data_ptr(), rows,
                          cols, hip_stream));
  NDArray::MarkUsedBy({p, l, loss}, stream);
}

void NLLLossGradientCuda(const NDArray& pred, const NDArray& label, const NDArray& grad_loss, NDArray& output,
                         const Stream& stream) {
  HT_ASSERT_CUDA_DEVICE(pred);
  HT_ASSERT_SAME_DEVICE(pred, label);
  HT_ASSERT_SAME_DEVICE(pred, grad_loss);
  HT_ASSERT_SAME_DEVICE(pred, output);
  HT_ASSERT_SAME_SHAPE(pred, output);
  HT_ASSERT_SAME_DTYPE(pred, output);
  HT_ASSERT_SAME_DTYPE(pred, grad_loss);
  HT_ASSERT(label->dtype() == kInt64) << "labels must be int64 class ids, got " << label->dtype();
  HT_ASSERT(pred->ndim() >= 1);
  HT_ASSERT_CONTIGUOUS(output);
  int64_t rows = 1;
  for (size_t i = 0; i + 1 < pred->ndim(); ++i) rows *= pred->shape(i);
  const int64_t cols = pred->shape(pred->ndim() - 1);
  HT_ASSERT(int64_t(label->numel()) == rows && int64_t(grad_loss->numel()) == rows)
    << "labels " << label->shape() << " / grad_loss " << grad_loss->shape() << " must hold one value per row of "
    << pred->shape();
  if (rows == 0 || cols == 0) return;

  HIPStream hip_stream(stream);
  hip::DeviceGuard guard(hip_stream.device_id());
  NDArray l = Dense(label, stream), g = Dense(grad_loss, stream);
  HK_CALL(hk_nll_loss_bwd(int(pred->dtype()), l->data_ptr<int64_t>(), g->raw_data_ptr(), output->raw_data_ptr(), rows,
                          cols, hip_stream));
  NDArray::MarkUsedBy({l, g, output}, stream);
}

// Host twins (hetu/impl/kernel/NLLLoss.cc of the reference): loss[r] = -pred[r, label[r]] (0 for a label outside
// [0, cols)); the gradient is zero but for -grad_loss[r] * cols at the label's column, the factor being the
// reference's (NLLLoss.cu:24-41).
void NLLLossCpu(const NDArray& pred, const NDArray& label, NDArray& loss, const Stream& stream) {
  HT_ASSERT_CPU_DEVICE(pred);
  HT_ASSERT_SAME_DEVICE(pred, label);
  HT_ASSERT_SAME_DEVICE(pred, loss);
  HT_ASSERT_SAME_SHAPE(label, loss);
  HT_ASSERT_SAME_DTYPE(pred, loss);
  HT_ASSERT(label->dtype() == kInt64) << "labels must be int64 class ids, got " << label->dtype();
  HT_ASSERT(pred->ndim() == label->ndim() + 1);
  for (size_t i = 0; i < label->ndim(); i++) HT_ASSERT(pred->shape(i) == label->shape(i));
  HT_ASSERT_CONTIGUOUS(loss);
  int64_t rows = 1;
  for (size_t i = 0; i < label->ndim(); i++) rows *= label->shape(i);
  const int64_t cols = pred->shape(pred->ndim() - 1);
  if (rows == 0) return;
  HT_DISPATCH_FLOATING_TYPES(pred->dtype(), spec_t, "NLLLossCpu", [&]() {
    cpu::on_stream(stream, "NLLLossCpu", [=]() {
      NDArray p = Dense(pred, stream), l = Dense(label, stream);
      using A = typename cpu::Arith<spec_t>::type;
      const spec_t* pp = p->data_ptr<spec_t>();
      const int64_t* lp = l->data_ptr<int64_t>();
      spec_t* out = loss->data_ptr<spec_t>();
      for (int64_t r = 0; r < rows; ++r) {
        const int64_t lab = lp[r];
        const bool ok = lab >= 0 && lab < cols;
        cpu::st<spec_t, A>(out + r, ok ? -cpu::ld<spec_t, A>(pp + r * cols + lab) : A(0));
      }
    });
  });
}

void NLLLossGradientCpu(const NDArray& pred, const NDArray& label, const NDArray& grad_loss, NDArray& output,
                        const Stream& stream) {
  HT_ASSERT_CPU_DEVICE(pred);
  HT_ASSERT_SAME_DEVICE(pred, label);
  HT_ASSERT_SAME_DEVICE(pred, grad_loss);
  HT_ASSERT_SAME_DEVICE(pred, output);
  HT_ASSERT_SAME_SHAPE(pred, output);
  HT_ASSERT_SAME_DTYPE(pred, output);
  HT_ASSERT_SAME_DTYPE(pred, grad_loss);
  HT_ASSERT(label->dtype() == kInt64) << "labels must be int64 class ids, got " << label->dtype();
  HT_ASSERT(pred->ndim() >= 1);
  HT_ASSERT_CONTIGUOUS(output);
  int64_t rows = 1;
  for (size_t i = 0; i + 1 < pred->ndim(); ++i) rows *= pred->shape(i);
  const int64_t cols = pred->shape(pred->ndim() - 1);
  HT_ASSERT(int64_t(label->numel()) == rows && int64_t(grad_loss->numel()) == rows)
    << "labels " << label->shape() << " / grad_loss " << grad_loss->shape() << " must hold one value per row of "
    << pred->shape();
  if (rows == 0 || cols == 0) return;
  HT_DISPATCH_FLOATING_TYPES(pred->dtype(), spec_t, "NLLLossGradientCpu", [&]() {
    cpu::on_stream(stream, "NLLLossGradientCpu", [=]() {
      NDArray l = Dense(label, stream), g = Dense(grad_loss, stream);
      using A = typename cpu::Arith<spec_t>::type;
      const int64_t* lp = l->data_ptr<int64_t>();
      const spec_t* gp = g->data_ptr<spec_t>();
      spec_t* out = output->data_ptr<spec_t>();
      cpu::parallel_rows(rows, cols, [&](int64_t r) {
        spec_t* dr = out + r * cols;
        for (int64_t c = 0; c < cols; ++c) cpu::st<spec_t, A>(dr + c, A(0));
        const int64_t lab = lp[r];
        if (lab >= 0 && lab < cols) cpu::st<spec_t, A>(dr + lab, -cpu::ld<spec_t, A>(gp + r) * A(cols));
      });
    });
  });
}

} // namespace impl
} // namespace hetu
