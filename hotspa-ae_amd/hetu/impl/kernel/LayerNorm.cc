// LayerNormCuda / LayerNormGradientCuda: same arguments and meaning as
// hetu/impl/kernel/LayerNorm.cu:66-121 and :235-337 of the reference (statistics
// are mean and VARIANCE, stored in the data dtype), run by the gfx950 kernels
// behind hk_layer_norm_fwd / hk_layer_norm_bwd.  The operator takes non-contiguous
// arrays (hetu/graph/ops/LayerNorm.h:78-80): row-pitched arrays and views with permuted
// leading dimensions go to the kernels as they are (RowPlan), any other layout through
// a dense copy (inputs) or a dense stand-in laid over the strides afterwards (outputs).
#include "hetu/graph/ops/kernel_links.h"
#include "hetu/impl/kernel/kernel_utils.h"
#include "hetu/impl/utils/cpu_utils.h"
#include "hetu/impl/utils/dispatch.h"

#include <algorithm>

namespace hetu {
namespace impl {

void LayerNormCuda(const NDArray& in_arr, const NDArray& ln_scale, const NDArray& ln_bias, NDArray& mean_arr,
                   NDArray& var_arr, NDArray& out_arr, int64_t reduce_dims, float eps, const Stream& stream) {
  HT_ASSERT_CUDA_DEVICE(in_arr);
  HT_ASSERT_SAME_DEVICE(in_arr, ln_scale);
  HT_ASSERT_SAME_DEVICE(in_arr, ln_bias);
  HT_ASSERT_SAME_DEVICE(in_arr, mean_arr);
  HT_ASSERT_SAME_DEVICE(in_arr, var_arr);
  HT_ASSERT_SAME_DEVICE(in_arr, out_arr);
  HT_ASSERT_SAME_SHAPE(in_arr, out_arr);
  HT_ASSERT_SAME_DTYPE(in_arr, out_arr);
  HT_ASSERT_SAME_DTYPE(in_arr, ln_scale);
  HT_ASSERT_SAME_DTYPE(in_arr, ln_bias);
  HT_ASSERT_SAME_DTYPE(in_arr, mean_arr);
  HT_ASSERT_SAME_DTYPE(in_arr, var_arr);
  HT_ASSERT_CONTIGUOUS(mean_arr);
  HT_ASSERT_CONTIGUOUS(var_arr);

  int64_t rows, cols;
  SplitRows(in_arr, reduce_dims, rows, cols);
  HT_ASSERT(int64_t(ln_scale->numel()) == cols && int64_t(ln_bias->numel()) == cols)
    << "scale " << ln_scale->shape() << " / bias " << ln_bias->shape() << " do not match " << cols << " columns";
  HT_ASSERT(int64_t(mean_arr->numel()) == rows && int64_t(var_arr->numel()) == rows)
    << "statistics must hold one value per row (" << rows << ")";
  if (in_arr->numel() == 0) return;

  HIPStream hip_stream(stream);
  hip::DeviceGuard guard(hip_stream.device_id());
  RowPlan plan(reduce_dims, stream);
  RowPlan::Slot& x = plan.Input(in_arr);
  RowPlan::Slot& y = plan.Output(out_arr);
  plan.Resolve();
  NDArray g = Dense(ln_scale, stream), b = Dense(ln_bias, stream);
  const int dt = int(in_arr->dtype());
  HK_CALL(hk_layer_norm_fwd_strided_rows(dt, x.ptr(), x.steps, g->raw_data_ptr(), b->raw_data_ptr(), y.ptr(), y.steps,
                                         mean_arr->raw_data_ptr(), var_arr->raw_data_ptr(), dt, HK_STAT_VAR,
                                         plan.level_rows(), cols, eps, hip_stream));
  NDArray::MarkUsedBy({x.array, g, b, mean_arr, var_arr, y.array}, stream);
  plan.Commit();
}

void LayerNormGradientCuda(const NDArray& out_grads, const NDArray& in_arr, const NDArray& ln_scale,
                           NDArray& grad_arr, NDArray& grad_scale, NDArray& grad_bias, const NDArray& mean_arr,
                           const NDArray& var_arr, int64_t reduce_dims, float eps, const Stream& stream) {
  HT_ASSERT_CUDA_DEVICE(out_grads);
  HT_ASSERT_SAME_DEVICE(out_grads, ln_scale);
  HT_ASSERT_SAME_DEVICE(out_grads, in_arr);
  HT_ASSERT_SAME_DEVICE(out_grads, mean_arr);
  HT_ASSERT_SAME_DEVICE(out_grads, var_arr);
  HT_ASSERT_SAME_DEVICE(out_grads, grad_scale);
  HT_ASSERT_SAME_DEVICE(out_grads, grad_arr);
  HT_ASSERT_SAME_DEVICE(out_grads, grad_bias);
  HT_ASSERT_SAME_SHAPE(out_grads, in_arr);
  HT_ASSERT_SAME_SHAPE(out_grads, grad_arr);
  HT_ASSERT_SAME_DTYPE(out_grads, in_arr);
  HT_ASSERT_SAME_DTYPE(out_grads, grad_arr);
  HT_ASSERT_SAME_DTYPE(out_grads, ln_scale);
  HT_ASSERT_SAME_DTYPE(out_grads, grad_scale);
  HT_ASSERT_SAME_DTYPE(out_grads, grad_bias);
  HT_ASSERT_SAME_DTYPE(out_grads, mean_arr);
  HT_ASSERT_SAME_DTYPE(out_grads, var_arr);
  HT_ASSERT_CONTIGUOUS(grad_scale);
  HT_ASSERT_CONTIGUOUS(grad_bias);

  int64_t rows, cols;
  SplitRows(in_arr, reduce_dims, rows, cols);
  HT_ASSERT(int64_t(ln_scale->numel()) == cols && int64_t(grad_scale->numel()) == cols &&
            int64_t(grad_bias->numel()) == cols)
    << "scale / grad_scale / grad_bias must hold " << cols << " values";
  HT_ASSERT(int64_t(mean_arr->numel()) == rows && int64_t(var_arr->numel()) == rows)
    << "statistics must hold one value per row (" << rows << ")";

  HIPStream hip_stream(stream);
  hip::DeviceGuard guard(hip_stream.device_id());
  const int dt = int(in_arr->dtype());
  if (in_arr->numel() == 0) {
    // no rows: the column sums are empty sums
    const size_t bytes = size_t(cols) * DataType2Size(in_arr->dtype());
    if (bytes) {
      HK_CALL(hk_memset(grad_scale->raw_data_ptr(), 0, bytes, hip_stream));
      HK_CALL(hk_memset(grad_bias->raw_data_ptr(), 0, bytes, hip_stream));
      NDArray::MarkUsedBy({grad_scale, grad_bias}, stream);
    }
    return;
  }
  RowPlan plan(reduce_dims, stream);
  RowPlan::Slot& dy = plan.Input(out_grads);
  RowPlan::Slot& x = plan.Input(in_arr);
  RowPlan::Slot& dx = plan.Output(grad_arr);
  plan.Resolve();
  NDArray g = Dense(ln_scale, stream);
  NDArray mean = Dense(mean_arr, stream), var = Dense(var_arr, stream);
  size_t ws_bytes = 0;
  HK_CALL(hk_norm_bwd_workspace_bytes(dt, rows, cols, &ws_bytes));
  NDArray ws = Scratch(ws_bytes, in_arr->device(), stream);
  HK_CALL(hk_layer_norm_bwd_strided_rows(dt, dy.ptr(), dy.steps, x.ptr(), x.steps, g->raw_data_ptr(),
                                         /*beta=*/nullptr, mean->raw_data_ptr(), var->raw_data_ptr(), dt,
                                         HK_STAT_VAR, dx.ptr(), dx.steps, grad_scale->raw_data_ptr(),
                                         grad_bias->raw_data_ptr(), plan.level_rows(), cols, eps,
                                         /*memory_efficient=*/0, /*clamp_gamma=*/0, MutPtrOrNull(ws), ws_bytes,
                                         hip_stream));
  NDArray::MarkUsedBy({dy.array, x.array, g, mean, var, dx.array, grad_scale, grad_bias, ws}, stream);
  plan.Commit();
}

// ---------------------------------------------------------------------------------------------------------
// Host twins (hetu/impl/kernel/LayerNorm.cc:34-142 and :177-364 of the reference): the same three passes over a
// row as the reference makes over the array (mean; mean of (x - mean)^2; the output), and for the gradient the
// column sums first (grad_bias = sum dy, grad_scale = sum dy * x_hat) and then dx from the two row sums.  The
// reference's host dx leaves the scale out of the row terms (calculate_grad_kernel, LayerNorm.cc:160-175, never
// reads ln_scale); this twin computes what the accelerator kernel computes,
//   t = dy * scale,  dx = rstd * (t - mean(t) - x_hat * mean(t * x_hat)).
// The work runs in the calling thread (and its OpenMP team) before the call returns.
// ---------------------------------------------------------------------------------------------------------
void LayerNormCpu(const NDArray& in_arr, const NDArray& ln_scale, const NDArray& ln_bias, NDArray& mean_arr,
                  NDArray& var_arr, NDArray& out_arr, int64_t reduce_dims, float eps, const Stream& stream) {
  HT_ASSERT_CPU_DEVICE(in_arr);
  HT_ASSERT_SAME_DEVICE(in_arr, ln_scale);
  HT_ASSERT_SAME_DEVICE(in_arr, ln_bias);
  HT_ASSERT_SAME_DEVICE(in_arr, mean_arr);
  HT_ASSERT_SAME_DEVICE(in_arr, var_arr);
  HT_ASSERT_SAME_DEVICE(in_arr, out_arr);
  HT_ASSERT_SAME_SHAPE(in_arr, out_arr);
  HT_ASSERT_SAME_DTYPE(in_arr, out_arr);
  HT_ASSERT_SAME_DTYPE(in_arr, ln_scale);
  HT_ASSERT_SAME_DTYPE(in_arr, ln_bias);
  HT_ASSERT_SAME_DTYPE(in_arr, mean_arr);
  HT_ASSERT_SAME_DTYPE(in_arr, var_arr);
  HT_ASSERT_CONTIGUOUS(out_arr);
  HT_ASSERT_CONTIGUOUS(mean_arr);
  HT_ASSERT_CONTIGUOUS(var_arr);
  int64_t rows, cols;
  SplitRows(in_arr, reduce_dims, rows, cols);
  HT_ASSERT(int64_t(ln_scale->numel()) == cols && int64_t(ln_bias->numel()) == cols)
    << "scale / bias must hold " << cols << " values";
  HT_ASSERT(int64_t(mean_arr->numel()) == rows && int64_t(var_arr->numel()) == rows)
    << "statistics must hold one value per row (" << rows << ")";
  if (in_arr->numel() == 0) return;
  HT_DISPATCH_FLOATING_TYPES(in_arr->dtype(), spec_t, "LayerNormCpu", [&]() {
    cpu::on_stream(stream, "LayerNormCpu", [=]() {
      NDArray x = Dense(in_arr, stream), g = Dense(ln_scale, stream), b = Dense(ln_bias, stream);
      using A = typename cpu::Arith<spec_t>::type;
      const spec_t* xp = x->data_ptr<spec_t>();
      const spec_t* gp = g->data_ptr<spec_t>();
      const spec_t* bp = b->data_ptr<spec_t>();
      spec_t* mp = mean_arr->data_ptr<spec_t>();
      spec_t* vp = var_arr->data_ptr<spec_t>();
      spec_t* yp = out_arr->data_ptr<spec_t>();
      const A inv = A(1) / A(cols);
      cpu::parallel_rows(rows, cols, [&](int64_t r) {
        const spec_t* xr = xp + r * cols;
        const A mean = cpu::blocked_sum<A>(cols, [&](int64_t i) { return cpu::ld<spec_t, A>(xr + i); }) * inv;
        const A var = cpu::blocked_sum<A>(cols, [&](int64_t i) {
          const A d = cpu::ld<spec_t, A>(xr + i) - mean;
          return d * d;
        }) * inv;
        cpu::st<spec_t, A>(mp + r, mean);
        cpu::st<spec_t, A>(vp + r, var);
        const A rstd = A(1) / std::sqrt(var + A(eps));
        spec_t* yr = yp + r * cols;
        cpu::for_range(0, cols, [&](int64_t i) {
          cpu::st<spec_t, A>(yr + i, (cpu::ld<spec_t, A>(xr + i) - mean) * rstd * cpu::ld<spec_t, A>(gp + i) +
                                       cpu::ld<spec_t, A>(bp + i));
        });
      });
    });
  });
}

void LayerNormGradientCpu(const NDArray& out_grads, const NDArray& in_arr, const NDArray& ln_scale,
                          NDArray& grad_arr, NDArray& grad_scale, NDArray& grad_bias, const NDArray& mean_arr,
                          const NDArray& var_arr, int64_t reduce_dims, float eps, const Stream& stream) {
  HT_ASSERT_CPU_DEVICE(out_grads);
  HT_ASSERT_SAME_DEVICE(out_grads, ln_scale);
  HT_ASSERT_SAME_DEVICE(out_grads, in_arr);
  HT_ASSERT_SAME_DEVICE(out_grads, mean_arr);
  HT_ASSERT_SAME_DEVICE(out_grads, var_arr);
  HT_ASSERT_SAME_DEVICE(out_grads, grad_scale);
  HT_ASSERT_SAME_DEVICE(out_grads, grad_arr);
  HT_ASSERT_SAME_DEVICE(out_grads, grad_bias);
  HT_ASSERT_SAME_SHAPE(out_grads, in_arr);
  HT_ASSERT_SAME_SHAPE(out_grads, grad_arr);
  HT_ASSERT_SAME_DTYPE(out_grads, in_arr);
  HT_ASSERT_SAME_DTYPE(out_grads, grad_arr);
  HT_ASSERT_SAME_DTYPE(out_grads, ln_scale);
  HT_ASSERT_SAME_DTYPE(out_grads, grad_scale);
  HT_ASSERT_SAME_DTYPE(out_grads, grad_bias);
  HT_ASSERT_SAME_DTYPE(out_grads, mean_arr);
  HT_ASSERT_SAME_DTYPE(out_grads, var_arr);
  HT_ASSERT_CONTIGUOUS(grad_arr);
  HT_ASSERT_CONTIGUOUS(grad_scale);
  HT_ASSERT_CONTIGUOUS(grad_bias);
  int64_t rows, cols;
  SplitRows(in_arr, reduce_dims, rows, cols);
  HT_ASSERT(int64_t(ln_scale->numel()) == cols && int64_t(grad_scale->numel()) == cols &&
            int64_t(grad_bias->numel()) == cols)
    << "scale / grad_scale / grad_bias must hold " << cols << " values";
  HT_ASSERT(int64_t(mean_arr->numel()) == rows && int64_t(var_arr->numel()) == rows)
    << "statistics must hold one value per row (" << rows << ")";
  HT_DISPATCH_FLOATING_TYPES(in_arr->dtype(), spec_t, "LayerNormGradientCpu", [&]() {
    cpu::on_stream(stream, "LayerNormGradientCpu", [=]() {
      NDArray dy = Dense(out_grads, stream), x = Dense(in_arr, stream), g = Dense(ln_scale, stream);
      NDArray mean = Dense(mean_arr, stream), var = Dense(var_arr, stream);
      using A = typename cpu::Arith<spec_t>::type;
      const spec_t* dyp = dy->data_ptr<spec_t>();
      const spec_t* xp = x->data_ptr<spec_t>();
      const spec_t* gp = g->data_ptr<spec_t>();
      const spec_t* mp = mean->data_ptr<spec_t>();
      const spec_t* vp = var->data_ptr<spec_t>();
      spec_t* dxp = grad_arr->data_ptr<spec_t>();
      spec_t* dgp = grad_scale->data_ptr<spec_t>();
      spec_t* dbp = grad_bias->data_ptr<spec_t>();
      // column sums, a band of columns per thread: every thread walks all rows of its band
      constexpr int64_t kBand = 64;
      const int64_t bands = (cols + kBand - 1) / kBand;
      cpu::parallel_rows(bands, rows * kBand, [&](int64_t band) {
        const int64_t c0 = band * kBand, c1 = std::min(cols, c0 + kBand);
        A sg[kBand], sb[kBand];
        for (int64_t c = 0; c < kBand; ++c) sg[c] = sb[c] = A(0);
        for (int64_t r = 0; r < rows; ++r) {
          const A m = cpu::ld<spec_t, A>(mp + r);
          const A rstd = A(1) / std::sqrt(cpu::ld<spec_t, A>(vp + r) + A(eps));
          const spec_t* dyr = dyp + r * cols;
          const spec_t* xr = xp + r * cols;
          cpu::for_range(c0, c1, [&](int64_t c) {
            const A d = cpu::ld<spec_t, A>(dyr + c);
            sb[c - c0] += d;
            sg[c - c0] += d * (cpu::ld<spec_t, A>(xr + c) - m) * rstd;
          });
        }
        for (int64_t c = c0; c < c1; ++c) {
          cpu::st<spec_t, A>(dgp + c, sg[c - c0]);
          cpu::st<spec_t, A>(dbp + c, sb[c - c0]);
        }
      });
      if (in_arr->numel() == 0) return;
      const A inv = A(1) / A(cols);
      cpu::parallel_rows(rows, cols, [&](int64_t r) {
        const A m = cpu::ld<spec_t, A>(mp + r);
        const A rstd = A(1) / std::sqrt(cpu::ld<spec_t, A>(vp + r) + A(eps));
        const spec_t* dyr = dyp + r * cols;
        const spec_t* xr = xp + r * cols;
        const A s1 = cpu::blocked_sum<A>(cols, [&](int64_t i) {
          return cpu::ld<spec_t, A>(dyr + i) * cpu::ld<spec_t, A>(gp + i);
        }) * inv;
        const A s2 = cpu::blocked_sum<A>(cols, [&](int64_t i) {
          return cpu::ld<spec_t, A>(dyr + i) * cpu::ld<spec_t, A>(gp + i) * (cpu::ld<spec_t, A>(xr + i) - m) * rstd;
        }) * inv;
        spec_t* dxr = dxp + r * cols;
        cpu::for_range(0, cols, [&](int64_t i) {
          const A xh = (cpu::ld<spec_t, A>(xr + i) - m) * rstd;
          const A t = cpu::ld<spec_t, A>(dyr + i) * cpu::ld<spec_t, A>(gp + i);
          cpu::st<spec_t, A>(dxr + i, rstd * (t - s1 - xh * s2));
        });
      });
    });
  });
}

} // namespace impl
} // namespace hetu
