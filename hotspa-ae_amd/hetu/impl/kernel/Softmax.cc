// SoftmaxCuda / SoftmaxGradientCuda: arguments and meaning of
// hetu/impl/kernel/Softmax.cu:250-310 and :364-404 of the reference.  The array
// is seen as [outer, dim, inner].  The operator takes non-contiguous arrays
// (hetu/graph/ops/Softmax.h:52-54): for a softmax over the last dimension row-pitched
// inputs and outputs go to the kernels as they are; any other input layout is made
// dense first, any other output layout is written dense and laid over its strides
// afterwards (RowOutput), as is the output of a softmax over another dimension.
#include "hetu/graph/ops/kernel_links.h"
#include "hetu/impl/kernel/kernel_utils.h"
#include "hetu/impl/utils/cpu_utils.h"
#include "hetu/impl/utils/dispatch.h"

namespace hetu {
namespace impl {

namespace {
void SplitAtDim(const NDArray& a, int64_t& dim, int64_t& outer, int64_t& extent, int64_t& inner) {
  dim = NDArrayMeta::ParseAxis(dim, int64_t(a->ndim()));
  outer = inner = 1;
  extent = a->shape(dim);
  for (int64_t i = 0; i < int64_t(a->ndim()); ++i) {
    if (i < dim) outer *= a->shape(i);
    else if (i > dim) inner *= a->shape(i);
  }
}
} // namespace

void SoftmaxCuda(const NDArray& input, NDArray& output, int64_t dim, const Stream& stream) {
  HT_ASSERT_CUDA_DEVICE(input);
  HT_ASSERT_SAME_DEVICE(input, output);
  HT_ASSERT_SAME_SHAPE(input, output);
  HT_ASSERT_SAME_DTYPE(input, output);
  int64_t outer, extent, inner;
  SplitAtDim(input, dim, outer, extent, inner);
  if (input->numel() == 0) return;

  HIPStream hip_stream(stream);
  hip::DeviceGuard guard(hip_stream.device_id());
  if (inner == 1) {
    // row-pitched arrays and views with permuted leading dimensions are read and written in place
    RowPlan plan(1, stream);
    RowPlan::Slot& x = plan.Input(input);
    RowPlan::Slot& y = plan.Output(output);
    plan.Resolve(/*vector_rows_only=*/true);
    HK_CALL(hk_softmax_fwd_strided_rows(int(input->dtype()), x.ptr(), x.steps, y.ptr(), y.steps, plan.level_rows(),
                                        extent, hip_stream));
    NDArray::MarkUsedBy({x.array, y.array}, stream);
    plan.Commit();
    return;
  }
  NDArray x = Dense(input, stream);
  RowOutput y(output, -1, stream);
  HK_CALL(hk_softmax_fwd(int(input->dtype()), x->raw_data_ptr(), y.ptr(), outer, extent, inner, hip_stream));
  NDArray::MarkUsedBy({x, y.array()}, stream);
  y.Commit();
}

void SoftmaxGradientCuda(const NDArray& input_Y, const NDArray& output_grad, NDArray& input_grad, int64_t dim,
                         const Stream& stream) {
  HT_ASSERT_CUDA_DEVICE(input_Y);
  HT_ASSERT_SAME_DEVICE(input_Y, output_grad);
  HT_ASSERT_SAME_DEVICE(input_Y, input_grad);
  HT_ASSERT_SAME_SHAPE(input_Y, output_grad);
  HT_ASSERT_SAME_SHAPE(input_Y, input_grad);
  HT_ASSERT_SAME_DTYPE(input_Y, output_grad);
  HT_ASSERT_SAME_DTYPE(input_Y, input_grad);
  int64_t outer, extent, inner;
  SplitAtDim(input_Y, dim, outer, extent, inner);
  if (input_Y->numel() == 0) return;

  HIPStream hip_stream(stream);
  hip::DeviceGuard guard(hip_stream.device_id());
  if (inner == 1) {
    RowPlan plan(1, stream);
    RowPlan::Slot& y = plan.Input(input_Y);
    RowPlan::Slot& dy = plan.Input(output_grad);
    RowPlan::Slot& dx = plan.Output(input_grad);
    plan.Resolve(/*vector_rows_only=*/true);
    HK_CALL(hk_softmax_bwd_strided_rows(int(input_Y->dtype()), y.ptr(), y.steps, dy.ptr(), dy.steps, dx.ptr(), dx.steps,
                                        plan.level_rows(), extent, hip_stream));
    NDArray::MarkUsedBy({y.array, dy.array, dx.array}, stream);
    plan.Commit();
    return;
  }
  NDArray y = Dense(input_Y, stream), dy = Dense(output_grad, stream);
  RowOutput dx(input_grad, -1, stream);
  HK_CALL(hk_softmax_bwd(int(input_Y->dtype()), y->raw_data_ptr(), dy->raw_data_ptr(), dx.ptr(), outer, extent, inner,
                         hip_stream));
  NDArray::MarkUsedBy({y, dy, dx.array()}, stream);
  dx.Commit();
}

// ---------------------------------------------------------------------------------------------------------
// Host twins (hetu/impl/kernel/Softmax.cc:11-97 of the reference, oneDNN's softmax_accurate there): per line
// along `dim` the maximum, the sum of exp(x - max), then exp(x - max) / sum; for the gradient
// dx = y * (dy - sum(dy * y)).  Lines are independent and shared out over the OpenMP team.
// ---------------------------------------------------------------------------------------------------------
void SoftmaxCpu(const NDArray& input, NDArray& output, int64_t dim, const Stream& stream) {
  HT_ASSERT_CPU_DEVICE(input);
  HT_ASSERT_SAME_DEVICE(input, output);
  HT_ASSERT_SAME_SHAPE(input, output);
  HT_ASSERT_SAME_DTYPE(input, output);
  HT_ASSERT_CONTIGUOUS(output);
  int64_t outer, extent, inner;
  SplitAtDim(input, dim, outer, extent, inner);
  if (input->numel() == 0) return;
  HT_DISPATCH_FLOATING_TYPES(input->dtype(), spec_t, "SoftmaxCpu", [&]() {
    cpu::on_stream(stream, "SoftmaxCpu", [=]() {
      NDArray x = Dense(input, stream);
      using A = typename cpu::Arith<spec_t>::type;
      const spec_t* xp = x->data_ptr<spec_t>();
      spec_t* yp = output->data_ptr<spec_t>();
      cpu::with_step(inner, [&](auto step) {
        cpu::parallel_rows(outer * inner, extent, [&](int64_t line) {
          const int64_t o = line / inner, i = line - o * inner;
          const spec_t* xl = xp + o * extent * inner + i;
          spec_t* yl = yp + o * extent * inner + i;
          const A m = cpu::blocked_max<A>(extent, [&](int64_t k) { return cpu::ld<spec_t, A>(xl + k * step()); });
          // a line of -inf only: exp(-inf - -inf) is NaN, as on the accelerator
          const A sum = cpu::blocked_sum<A>(extent, [&](int64_t k) {
            return cpu::exp_(cpu::ld<spec_t, A>(xl + k * step()) - m);
          });
          const A inv = A(1) / sum;
          cpu::for_range(0, extent, [&](int64_t k) {
            cpu::st<spec_t, A>(yl + k * step(), cpu::exp_(cpu::ld<spec_t, A>(xl + k * step()) - m) * inv);
          });
        });
      });
    });
  });
}

void SoftmaxGradientCpu(const NDArray& input_Y, const NDArray& output_grad, NDArray& input_grad, int64_t dim,
                        const Stream& stream) {
  HT_ASSERT_CPU_DEVICE(input_Y);
  HT_ASSERT_SAME_DEVICE(input_Y, output_grad);
  HT_ASSERT_SAME_DEVICE(input_Y, input_grad);
  HT_ASSERT_SAME_SHAPE(input_Y, output_grad);
  HT_ASSERT_SAME_SHAPE(input_Y, input_grad);
  HT_ASSERT_SAME_DTYPE(input_Y, output_grad);
  HT_ASSERT_SAME_DTYPE(input_Y, input_grad);
  HT_ASSERT_CONTIGUOUS(input_grad);
  int64_t outer, extent, inner;
  SplitAtDim(input_Y, dim, outer, extent, inner);
  if (input_Y->numel() == 0) return;
  HT_DISPATCH_FLOATING_TYPES(input_Y->dtype(), spec_t, "SoftmaxGradientCpu", [&]() {
    cpu::on_stream(stream, "SoftmaxGradientCpu", [=]() {
      NDArray y = Dense(input_Y, stream), dy = Dense(output_grad, stream);
      using A = typename cpu::Arith<spec_t>::type;
      const spec_t* yp = y->data_ptr<spec_t>();
      const spec_t* dyp = dy->data_ptr<spec_t>();
      spec_t* dxp = input_grad->data_ptr<spec_t>();
      cpu::with_step(inner, [&](auto step) {
        cpu::parallel_rows(outer * inner, extent, [&](int64_t line) {
          const int64_t o = line / inner, i = line - o * inner;
          const spec_t* yl = yp + o * extent * inner + i;
          const spec_t* dyl = dyp + o * extent * inner + i;
          spec_t* dxl = dxp + o * extent * inner + i;
          const A dot = cpu::blocked_sum<A>(extent, [&](int64_t k) {
            return cpu::ld<spec_t, A>(yl + k * step()) * cpu::ld<spec_t, A>(dyl + k * step());
          });
          cpu::for_range(0, extent, [&](int64_t k) {
            cpu::st<spec_t, A>(dxl + k * step(),
                               cpu::ld<spec_t, A>(yl + k * step()) * (cpu::ld<spec_t, A>(dyl + k * step()) - dot));
          });
        });
      });
    });
  });
}

} // namespace impl
} // namespace hetu
