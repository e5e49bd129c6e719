// SoftmaxCrossEntropySparseCuda / ...GradientCuda: arguments and meaning of
// hetu/impl/kernel/SoftmaxCrossEntropySparse.cu:239-274 and :276-318 of the
// reference.  Labels are int64 class ids, one per row; a row whose label equals
// `ignored_index` has loss 0 and a zero gradient row.
#include "hetu/graph/ops/kernel_links.h"
#include "hetu/impl/kernel/kernel_utils.h"
#include "hetu/impl/utils/cpu_utils.h"
#include "hetu/impl/utils/dispatch.h"

namespace hetu {
namespace impl {

namespace {
void RowsCols(const NDArray& pred, int64_t& rows, int64_t& cols) {
  HT_ASSERT(pred->ndim() >= 1) << "predictions need at least one dimension";
  rows = 1;
  for (size_t i = 0; i + 1 < pred->ndim(); ++i) rows *= pred->shape(i);
  cols = pred->shape(pred->ndim() - 1);
}
} // namespace

void SoftmaxCrossEntropySparseCuda(const NDArray& pred, const NDArray& label, NDArray& loss,
                                   const int64_t ignored_index, const Stream& stream) {
  HT_ASSERT_CUDA_DEVICE(pred);
  HT_ASSERT_SAME_DEVICE(pred, label);
  HT_ASSERT_SAME_DEVICE(pred, loss);
  HT_ASSERT_SAME_DTYPE(pred, loss);
  HT_ASSERT(label->dtype() == kInt64) << "labels must be int64 class ids, got " << label->dtype();
  HT_ASSERT_CONTIGUOUS(loss);
  int64_t rows, cols;
  RowsCols(pred, rows, cols);
  HT_ASSERT(int64_t(label->numel()) == rows && int64_t(loss->numel()) == rows)
    << "labels " << label->shape() << " / loss " << loss->shape() << " must hold one value per row of "
    << pred->shape();
  if (rows == 0) return;
  HT_VALUE_ERROR_IF(cols == 0) << "cross entropy over zero classes";

  HIPStream hip_stream(stream);
  hip::DeviceGuard guard(hip_stream.device_id());
  // row-pitched logits and views with permuted leading dimensions are read in place
  RowPlan plan(1, stream);
  RowPlan::Slot& p = plan.Input(pred);
  plan.Resolve();
  NDArray l = Dense(label, stream);
  HK_CALL(hk_sce_sparse_fwd_strided_rows(int(pred->dtype()), p.ptr(), p.steps, l->data_ptr<int64_t>(),
                                         loss->raw_data_ptr(), plan.level_rows(), cols, ignored_index, hip_stream));
  NDArray::MarkUsedBy({p.array, l, loss}, stream);
}

namespace {
// scale == nullptr: grad_loss holds one value per row; else it holds ONE value, used as
// round(grad_loss[0] * round(*scale)) by every row
void SparseGradient(const NDArray& pred, const NDArray& label, const NDArray& grad_loss, const double* scale,
                    NDArray& output, const int64_t ignored_index, const Stream& stream) {
  HT_ASSERT_CUDA_DEVICE(pred);
  HT_ASSERT_SAME_DEVICE(pred, label);
  HT_ASSERT_SAME_DEVICE(pred, grad_loss);
  HT_ASSERT_SAME_DEVICE(pred, output);
  HT_ASSERT_SAME_SHAPE(pred, output);
  HT_ASSERT_SAME_DTYPE(pred, output);
  HT_ASSERT_SAME_DTYPE(pred, grad_loss);
  HT_ASSERT(label->dtype() == kInt64) << "labels must be int64 class ids, got " << label->dtype();
  int64_t rows, cols;
  RowsCols(pred, rows, cols);
  HT_ASSERT(int64_t(label->numel()) == rows) << "labels " << label->shape() << " must hold one value per row of "
                                             << pred->shape();
  if (scale) {
    HT_ASSERT(grad_loss->numel() == 1) << "the gradient of a reduced loss is one value, got " << grad_loss->shape();
  } else {
    HT_ASSERT(int64_t(grad_loss->numel()) == rows)
      << "labels " << label->shape() << " / grad_loss " << grad_loss->shape() << " must hold one value per row of "
      << pred->shape();
  }
  if (rows == 0 || cols == 0) return;

  HIPStream hip_stream(stream);
  hip::DeviceGuard guard(hip_stream.device_id());
  NDArray l = Dense(label, stream), g = Dense(grad_loss, stream);
  if (scale) {
    NDArray p = Dense(pred, stream);
    RowOutput out(output, -1, stream);
    HK_CALL(hk_sce_sparse_bwd_reduced(int(pred->dtype()), p->raw_data_ptr(), l->data_ptr<int64_t>(),
                                      g->raw_data_ptr(), *scale, out.ptr(), rows, cols, ignored_index,
                                      hip_stream));
    NDArray::MarkUsedBy({p, l, g, out.array()}, stream);
    out.Commit();
    return;
  }
  // row-pitched arrays and views with permuted leading dimensions are read and written in place
  RowPlan plan(1, stream);
  RowPlan::Slot& p = plan.Input(pred);
  RowPlan::Slot& out = plan.Output(output);
  plan.Resolve();
  HK_CALL(hk_sce_sparse_bwd_strided_rows(int(pred->dtype()), p.ptr(), p.steps, l->data_ptr<int64_t>(),
                                         g->raw_data_ptr(), out.ptr(), out.steps, plan.level_rows(), cols,
                                         ignored_index, hip_stream));
  NDArray::MarkUsedBy({p.array, l, g, out.array}, stream);
  plan.Commit();
}
} // namespace

void SoftmaxCrossEntropySparseGradientCuda(const NDArray& pred, const NDArray& label, const NDArray& grad_loss,
                                           NDArray& output, const int64_t ignored_index, const Stream& stream) {
  SparseGradient(pred, label, grad_loss, nullptr, output, ignored_index, stream);
}

// No counterpart in the reference, whose gradient op first broadcasts the one gradient value times `scale`
// into a [rows] array (hetu/graph/ops/SoftmaxCrossEntropySparse.cc:64-85) and then calls the kernel above.
void SoftmaxCrossEntropySparseGradientReducedCuda(const NDArray& pred, const NDArray& label,
                                                  const NDArray& grad_output, double scale, NDArray& output,
                                                  const int64_t ignored_index, const Stream& stream) {
  SparseGradient(pred, label, grad_output, &scale, output, ignored_index, stream);
}

// ---------------------------------------------------------------------------------------------------------
// Host twins (hetu/impl/kernel/SoftmaxCrossEntropySparse.cc:11-126 of the reference): per row the maximum, the sum
// of exp(x - max), then loss = log(sum) - (x[label] - max), or the gradient (softmax - onehot) * grad_loss.  A row
// whose label is `ignored_index` gets loss 0 / a zero gradient row and the other rows are still computed (the
// reference's loops leave the whole parallel chunk at the first such row, SoftmaxCrossEntropySparse.cc:21-24,
// 47-53); a label outside [0, cols) gives NaN, as on the accelerator.
// ---------------------------------------------------------------------------------------------------------
void SoftmaxCrossEntropySparseCpu(const NDArray& pred, const NDArray& label, NDArray& loss,
                                  const int64_t ignored_index, const Stream& stream) {
  HT_ASSERT_CPU_DEVICE(pred);
  HT_ASSERT_SAME_DEVICE(pred, label);
  HT_ASSERT_SAME_DEVICE(pred, loss);
  HT_ASSERT_SAME_DTYPE(pred, loss);
  HT_ASSERT(label->dtype() == kInt64) << "labels must be int64 class ids, got " << label->dtype();
  HT_ASSERT_CONTIGUOUS(loss);
  int64_t rows, cols;
  RowsCols(pred, rows, cols);
  HT_ASSERT(int64_t(label->numel()) == rows && int64_t(loss->numel()) == rows)
    << "labels " << label->shape() << " / loss " << loss->shape() << " must hold one value per row of "
    << pred->shape();
  if (rows == 0) return;
  HT_VALUE_ERROR_IF(cols == 0) << "cross entropy over zero classes";
  HT_DISPATCH_FLOATING_TYPES(pred->dtype(), spec_t, "SoftmaxCrossEntropySparseCpu", [&]() {
    cpu::on_stream(stream, "SoftmaxCrossEntropySparseCpu", [=]() {
      NDArray p = Dense(pred, stream), l = Dense(label, stream);
      using A = typename cpu::Arith<spec_t>::type;
      const spec_t* pp = p->data_ptr<spec_t>();
      const int64_t* lp = l->data_ptr<int64_t>();
      spec_t* out = loss->data_ptr<spec_t>();
      cpu::parallel_rows(rows, cols, [&](int64_t r) {
        const int64_t lab = lp[r];
        if (lab == ignored_index) { cpu::st<spec_t, A>(out + r, A(0)); return; }
        if (lab < 0 || lab >= cols) { cpu::st<spec_t, A>(out + r, std::numeric_limits<A>::quiet_NaN()); return; }
        const spec_t* xr = pp + r * cols;
        const A m = cpu::blocked_max<A>(cols, [&](int64_t i) { return cpu::ld<spec_t, A>(xr + i); });
        const A sum = cpu::blocked_sum<A>(cols, [&](int64_t i) { return cpu::exp_(cpu::ld<spec_t, A>(xr + i) - m); });
        cpu::st<spec_t, A>(out + r, std::log(sum) - (cpu::ld<spec_t, A>(xr + lab) - m));
      });
    });
  });
}

void SoftmaxCrossEntropySparseGradientCpu(const NDArray& pred, const NDArray& label, const NDArray& grad_loss,
                                          NDArray& output, const int64_t ignored_index, const Stream& stream) {
  HT_ASSERT_CPU_DEVICE(pred);
  HT_ASSERT_SAME_DEVICE(pred, label);
  HT_ASSERT_SAME_DEVICE(pred, grad_loss);
  HT_ASSERT_SAME_DEVICE(pred, output);
  HT_ASSERT_SAME_SHAPE(pred, output);
  HT_ASSERT_SAME_DTYPE(pred, output);
  HT_ASSERT_SAME_DTYPE(pred, grad_loss);
  HT_ASSERT(label->dtype() == kInt64) << "labels must be int64 class ids, got " << label->dtype();
  HT_ASSERT_CONTIGUOUS(output);
  int64_t rows, cols;
  RowsCols(pred, rows, cols);
  HT_ASSERT(int64_t(label->numel()) == rows && int64_t(grad_loss->numel()) == rows)
    << "labels " << label->shape() << " / grad_loss " << grad_loss->shape()
    << " must hold one value per row of " << pred->shape();
  if (pred->numel() == 0) return;
  HT_DISPATCH_FLOATING_TYPES(pred->dtype(), spec_t, "SoftmaxCrossEntropySparseGradientCpu", [&]() {
    cpu::on_stream(stream, "SoftmaxCrossEntropySparseGradientCpu", [=]() {
      NDArray p = Dense(pred, stream), l = Dense(label, stream), gl = Dense(grad_loss, stream);
      using A = typename cpu::Arith<spec_t>::type;
      const spec_t* pp = p->data_ptr<spec_t>();
      const int64_t* lp = l->data_ptr<int64_t>();
      const spec_t* gp = gl->data_ptr<spec_t>();
      spec_t* out = output->data_ptr<spec_t>();
      cpu::parallel_rows(rows, cols, [&](int64_t r) {
        const int64_t lab = lp[r];
        spec_t* dr = out + r * cols;
        if (lab == ignored_index) {
          for (int64_t i = 0; i < cols; ++i) cpu::st<spec_t, A>(dr + i, A(0));
          return;
        }
        if (lab < 0 || lab >= cols) {
          for (int64_t i = 0; i < cols; ++i) cpu::st<spec_t, A>(dr + i, std::numeric_limits<A>::quiet_NaN());
          return;
        }
        const spec_t* xr = pp + r * cols;
        const A g = cpu::ld<spec_t, A>(gp + r);
        const A m = cpu::blocked_max<A>(cols, [&](int64_t i) { return cpu::ld<spec_t, A>(xr + i); });
        const A sum = cpu::blocked_sum<A>(cols, [&](int64_t i) { return cpu::exp_(cpu::ld<spec_t, A>(xr + i) - m); });
        const A scale = g / sum;
        // the row without its label term (a loop with nothing but arithmetic in it), then the one element again
        cpu::for_range(0, cols, [&](int64_t i) {
          cpu::st<spec_t, A>(dr + i, cpu::exp_(cpu::ld<spec_t, A>(xr + i) - m) * scale);
        });
        cpu::st<spec_t, A>(dr + lab, cpu::exp_(cpu::ld<spec_t, A>(xr + lab) - m) * scale - g);
      });
    });
  });
}

} // namespace impl
} // namespace hetu
