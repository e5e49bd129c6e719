// SoftmaxCrossEntropyCuda / ...GradientCuda (dense labels of the predictions'
// shape): arguments and meaning of hetu/impl/kernel/SoftmaxCrossEntropy.cu:13-73
// and :91-171 of the reference, as one fused pass instead of the reference's
// cuDNN softmax + elementwise + cuDNN reduce.
#include "hetu/graph/ops/kernel_links.h"
#include "hetu/impl/kernel/kernel_utils.h"
#include "hetu/impl/utils/cpu_utils.h"
#include "hetu/impl/utils/dispatch.h"

#include <cmath>
#include <limits>

namespace hetu {
namespace impl {

void SoftmaxCrossEntropyCuda(const NDArray& input, const NDArray& label, NDArray& output, const Stream& stream) {
  HT_ASSERT_CUDA_DEVICE(input);
  HT_ASSERT_SAME_DEVICE(input, label);
  HT_ASSERT_SAME_DEVICE(input, output);
  const size_t indim = input->ndim();
  HT_ASSERT(indim >= 1 && indim == label->ndim() && (indim == output->ndim() + 1 || (indim == 1 && output->ndim() == 1)))
    << "Indim is " << indim << ", Label dim is " << label->ndim() << ", Output dim is " << output->ndim();
  HT_ASSERT_SAME_SHAPE(input, label);
  HT_ASSERT_SAME_DTYPE(input, label);
  HT_ASSERT_SAME_DTYPE(input, output);
  HT_ASSERT_CONTIGUOUS(output);
  int64_t rows = 1;
  for (size_t i = 0; i + 1 < indim; ++i) rows *= input->shape(i);
  const int64_t cols = input->shape(indim - 1);
  HT_ASSERT(int64_t(output->numel()) == rows) << "loss " << output->shape() << " must hold one value per row";
  if (rows * cols == 0) return;

  HIPStream hip_stream(stream);
  hip::DeviceGuard guard(hip_stream.device_id());
  NDArray x = Dense(input, stream), l = Dense(label, stream);
  HK_CALL(hk_sce_dense_fwd(int(input->dtype()), x->raw_data_ptr(), l->raw_data_ptr(), output->raw_data_ptr(), rows,
                           cols, hip_stream));
  NDArray::MarkUsedBy({x, l, output}, stream);
}

namespace {
// scale == nullptr: grad holds one value per row; else it holds ONE value, used as
// round(grad[0] * round(*scale)) by every row
void DenseGradient(const NDArray& input_y, const NDArray& label, const NDArray& grad, const double* scale,
                   NDArray& output, const Stream& stream) {
  HT_ASSERT_CUDA_DEVICE(input_y);
  HT_ASSERT_SAME_DEVICE(input_y, label);
  HT_ASSERT_SAME_DEVICE(input_y, grad);
  HT_ASSERT_SAME_DEVICE(input_y, output);
  const size_t indim = input_y->ndim();
  HT_ASSERT(indim >= 1 && indim == label->ndim() && indim == output->ndim() &&
            (scale || indim == grad->ndim() + 1 || (indim == 1 && grad->ndim() == 1)))
    << "Indim is " << indim << ", Label dim is " << label->ndim() << ", Output dim is " << output->ndim();
  HT_ASSERT_SAME_SHAPE(input_y, label);
  HT_ASSERT_SAME_SHAPE(input_y, output);
  HT_ASSERT_SAME_DTYPE(input_y, label);
  HT_ASSERT_SAME_DTYPE(input_y, grad);
  HT_ASSERT_SAME_DTYPE(input_y, output);
  int64_t rows = 1;
  for (size_t i = 0; i + 1 < indim; ++i) rows *= input_y->shape(i);
  const int64_t cols = input_y->shape(indim - 1);
  if (scale) {
    HT_ASSERT(grad->numel() == 1) << "the gradient of a reduced loss is one value, got " << grad->shape();
  } else {
    HT_ASSERT(int64_t(grad->numel()) == rows) << "grad " << grad->shape() << " must hold one value per row";
  }
  if (rows * cols == 0) return;

  HIPStream hip_stream(stream);
  hip::DeviceGuard guard(hip_stream.device_id());
  NDArray x = Dense(input_y, stream), l = Dense(label, stream), g = Dense(grad, stream);
  RowOutput out(output, -1, stream);
  if (scale) {
    HK_CALL(hk_sce_dense_bwd_reduced(int(input_y->dtype()), x->raw_data_ptr(), l->raw_data_ptr(), g->raw_data_ptr(),
                                     *scale, out.ptr(), rows, cols, hip_stream));
  } else {
    HK_CALL(hk_sce_dense_bwd(int(input_y->dtype()), x->raw_data_ptr(), l->raw_data_ptr(), g->raw_data_ptr(),
                             out.ptr(), rows, cols, hip_stream));
  }
  NDArray::MarkUsedBy({x, l, g, out.array()}, stream);
  out.Commit();
}
} // namespace

void SoftmaxCrossEntropyGradientCuda(const NDArray& input_y, const NDArray& label, const NDArray& grad,
                                     NDArray& output, const Stream& stream) {
  DenseGradient(input_y, label, grad, nullptr, output, stream);
}

// No counterpart in the reference, whose gradient op first broadcasts the one gradient value times `scale`
// into a [rows] array (hetu/graph/ops/SoftmaxCrossEntropy.cc:59-80) and then calls the kernel above.
void SoftmaxCrossEntropyGradientReducedCuda(const NDArray& input_y, const NDArray& label, const NDArray& grad_output,
                                            double scale, NDArray& output, const Stream& stream) {
  DenseGradient(input_y, label, grad_output, &scale, output, stream);
}

// Host twins (hetu/impl/kernel/SoftmaxCrossEntropy.cc:12-45 and :90-125 of the reference): per row the maximum and
// the sum of exp(x - max); loss = -sum label * (x - max - log sum), gradient (softmax - label) * grad_loss.
void SoftmaxCrossEntropyCpu(const NDArray& input, const NDArray& label, NDArray& output, const Stream& stream) {
  HT_ASSERT_CPU_DEVICE(input);
  HT_ASSERT_SAME_DEVICE(input, label);
  HT_ASSERT_SAME_DEVICE(input, output);
  const size_t indim = input->ndim();
  HT_ASSERT(indim >= 1 && indim == label->ndim() && (indim == output->ndim() + 1 || (indim == 1 && output->ndim() == 1)))
    << "Indim is " << indim << ", Label dim is " << label->ndim() << ", Output dim is " << output->ndim();
  HT_ASSERT_SAME_SHAPE(input, label);
  HT_ASSERT_SAME_DTYPE(input, label);
  HT_ASSERT_SAME_DTYPE(input, output);
  HT_ASSERT_CONTIGUOUS(output);
  int64_t rows = 1;
  for (size_t i = 0; i + 1 < indim; ++i) rows *= input->shape(i);
  const int64_t cols = input->shape(indim - 1);
  HT_ASSERT(int64_t(output->numel()) == rows) << "loss " << output->shape() << " must hold one value per row";
  if (rows * cols == 0) return;
  HT_DISPATCH_FLOATING_TYPES(input->dtype(), spec_t, "SoftmaxCrossEntropyCpu", [&]() {
    cpu::on_stream(stream, "SoftmaxCrossEntropyCpu", [=]() {
      NDArray x = Dense(input, stream), l = Dense(label, stream);
      using A = typename cpu::Arith<spec_t>::type;
      const spec_t* xp = x->data_ptr<spec_t>();
      const spec_t* lp = l->data_ptr<spec_t>();
      spec_t* out = output->data_ptr<spec_t>();
      cpu::parallel_rows(rows, cols, [&](int64_t r) {
        const spec_t* xr = xp + r * cols;
        const spec_t* lr = lp + r * cols;
        const A m = cpu::blocked_max<A>(cols, [&](int64_t i) { return cpu::ld<spec_t, A>(xr + i); });
        const A sum = cpu::blocked_sum<A>(cols, [&](int64_t i) { return cpu::exp_(cpu::ld<spec_t, A>(xr + i) - m); });
        const A lse = m + std::log(sum);
        const A acc = cpu::blocked_sum<A>(cols, [&](int64_t i) {
          return cpu::ld<spec_t, A>(lr + i) * (lse - cpu::ld<spec_t, A>(xr + i));
        });
        cpu::st<spec_t, A>(out + r, acc);
      });
    });
  });
}

void SoftmaxCrossEntropyGradientCpu(const NDArray& input_y, const NDArray& label, const NDArray& grad,
                                    NDArray& output, const Stream& stream) {
  HT_ASSERT_CPU_DEVICE(input_y);
  HT_ASSERT_SAME_DEVICE(input_y, label);
  HT_ASSERT_SAME_DEVICE(input_y, grad);
  HT_ASSERT_SAME_DEVICE(input_y, output);
  HT_ASSERT_SAME_SHAPE(input_y, label);
  HT_ASSERT_SAME_SHAPE(input_y, output);
  HT_ASSERT_SAME_DTYPE(input_y, label);
  HT_ASSERT_SAME_DTYPE(input_y, grad);
  HT_ASSERT_SAME_DTYPE(input_y, output);
  HT_ASSERT_CONTIGUOUS(output);
  const size_t indim = input_y->ndim();
  HT_ASSERT(indim >= 1);
  int64_t rows = 1;
  for (size_t i = 0; i + 1 < indim; ++i) rows *= input_y->shape(i);
  const int64_t cols = input_y->shape(indim - 1);
  HT_ASSERT(int64_t(grad->numel()) == rows) << "grad " << grad->shape() << " must hold one value per row";
  if (rows * cols == 0) return;
  HT_DISPATCH_FLOATING_TYPES(input_y->dtype(), spec_t, "SoftmaxCrossEntropyGradientCpu", [&]() {
    cpu::on_stream(stream, "SoftmaxCrossEntropyGradientCpu", [=]() {
      NDArray x = Dense(input_y, stream), l = Dense(label, stream), g = Dense(grad, stream);
      using A = typename cpu::Arith<spec_t>::type;
      const spec_t* xp = x->data_ptr<spec_t>();
      const spec_t* lp = l->data_ptr<spec_t>();
      const spec_t* gp = g->data_ptr<spec_t>();
      spec_t* out = output->data_ptr<spec_t>();
      cpu::parallel_rows(rows, cols, [&](int64_t r) {
        const spec_t* xr = xp + r * cols;
        const spec_t* lr = lp + r * cols;
        spec_t* dr = out + r * cols;
        const A gr = cpu::ld<spec_t, A>(gp + r);
        const A m = cpu::blocked_max<A>(cols, [&](int64_t i) { return cpu::ld<spec_t, A>(xr + i); });
        const A sum = cpu::blocked_sum<A>(cols, [&](int64_t i) { return cpu::exp_(cpu::ld<spec_t, A>(xr + i) - m); });
        cpu::for_range(0, cols, [&](int64_t i) {
          cpu::st<spec_t, A>(dr + i, (cpu::exp_(cpu::ld<spec_t, A>(xr + i) - m) / sum - cpu::ld<spec_t, A>(lr + i)) * gr);
        });
      });
    });
  });
}

} // namespace impl
} // namespace hetu
