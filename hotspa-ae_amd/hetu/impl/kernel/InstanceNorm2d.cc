// InstanceNormCuda / InstanceNormGradientCuda: arguments and meaning of
// hetu/impl/kernel/InstanceNorm2d.cu:60-103 and :191-290 of the reference.  An
// instance norm of [N, C, H, W] is a layer norm without scale and bias over the
// H*W elements of each of the N*C planes, so both run on the layer-norm kernels
// (statistics are mean and variance in the data dtype, one per plane).
#include "hetu/graph/ops/kernel_links.h"
#include "hetu/impl/kernel/kernel_utils.h"
#include "hetu/impl/utils/cpu_utils.h"
#include "hetu/impl/utils/dispatch.h"

#include <cmath>

namespace hetu {
namespace impl {

namespace {
void Planes(const NDArray& in_arr, int64_t& rows, int64_t& cols) {
  HT_ASSERT(in_arr->ndim() == 4) << "instance norm expects [N, C, H, W], got " << in_arr->shape();
  rows = in_arr->shape(0) * in_arr->shape(1);
  cols = in_arr->shape(2) * in_arr->shape(3);
}
} // namespace

void InstanceNormCuda(const NDArray& in_arr, NDArray& mean_arr, NDArray& var_arr, NDArray& out_arr, float eps,
                      const Stream& stream) {
  HT_ASSERT_CUDA_DEVICE(in_arr);
  HT_ASSERT_SAME_DEVICE(in_arr, mean_arr);
  HT_ASSERT_SAME_DEVICE(in_arr, var_arr);
  HT_ASSERT_SAME_DEVICE(in_arr, out_arr);
  HT_ASSERT_SAME_SHAPE(in_arr, out_arr);
  HT_ASSERT_SAME_DTYPE(in_arr, out_arr);
  HT_ASSERT_SAME_DTYPE(in_arr, mean_arr);
  HT_ASSERT_SAME_DTYPE(in_arr, var_arr);
  HT_ASSERT_CONTIGUOUS(out_arr);
  HT_ASSERT_CONTIGUOUS(mean_arr);
  HT_ASSERT_CONTIGUOUS(var_arr);
  int64_t rows, cols;
  Planes(in_arr, rows, cols);
  HT_ASSERT(int64_t(mean_arr->numel()) == rows && int64_t(var_arr->numel()) == rows)
    << "statistics must hold one value per plane (" << rows << ")";
  if (in_arr->numel() == 0) return;

  HIPStream hip_stream(stream);
  hip::DeviceGuard guard(hip_stream.device_id());
  NDArray x = Dense(in_arr, stream);
  const int dt = int(in_arr->dtype());
  HK_CALL(hk_layer_norm_fwd(dt, x->raw_data_ptr(), /*gamma=*/nullptr, /*beta=*/nullptr, out_arr->raw_data_ptr(),
                            mean_arr->raw_data_ptr(), var_arr->raw_data_ptr(), dt, HK_STAT_VAR, rows, cols, eps,
                            hip_stream));
  NDArray::MarkUsedBy({x, mean_arr, var_arr, out_arr}, stream);
}

void InstanceNormGradientCuda(const NDArray& out_grads, const NDArray& in_arr, NDArray& grad_arr,
                              const NDArray& mean_arr, const NDArray& var_arr, float eps, const Stream& stream) {
  HT_ASSERT_CUDA_DEVICE(out_grads);
  HT_ASSERT_SAME_DEVICE(out_grads, in_arr);
  HT_ASSERT_SAME_DEVICE(out_grads, grad_arr);
  HT_ASSERT_SAME_DEVICE(out_grads, mean_arr);
  HT_ASSERT_SAME_DEVICE(out_grads, var_arr);
  HT_ASSERT_SAME_SHAPE(out_grads, in_arr);
  HT_ASSERT_SAME_SHAPE(out_grads, grad_arr);
  HT_ASSERT_SAME_DTYPE(out_grads, in_arr);
  HT_ASSERT_SAME_DTYPE(out_grads, grad_arr);
  HT_ASSERT_SAME_DTYPE(out_grads, mean_arr);
  HT_ASSERT_SAME_DTYPE(out_grads, var_arr);
  HT_ASSERT_CONTIGUOUS(grad_arr);
  int64_t rows, cols;
  Planes(in_arr, rows, cols);
  HT_ASSERT(int64_t(mean_arr->numel()) == rows && int64_t(var_arr->numel()) == rows)
    << "statistics must hold one value per plane (" << rows << ")";
  if (in_arr->numel() == 0) return;

  HIPStream hip_stream(stream);
  hip::DeviceGuard guard(hip_stream.device_id());
  NDArray dy = Dense(out_grads, stream), x = Dense(in_arr, stream);
  NDArray mean = Dense(mean_arr, stream), var = Dense(var_arr, stream);
  const int dt = int(in_arr->dtype());
  // no scale, no bias: nothing to sum over the planes, so no workspace either
  HK_CALL(hk_layer_norm_bwd(dt, dy->raw_data_ptr(), x->raw_data_ptr(), /*gamma=*/nullptr, /*beta=*/nullptr,
                            mean->raw_data_ptr(), var->raw_data_ptr(), dt, HK_STAT_VAR, grad_arr->raw_data_ptr(),
                            /*dgamma=*/nullptr, /*dbeta=*/nullptr, rows, cols, eps, /*memory_efficient=*/0,
                            /*clamp_gamma=*/0, /*workspace=*/nullptr, 0, hip_stream));
  NDArray::MarkUsedBy({dy, x, mean, var, grad_arr}, stream);
}

// Host twins (hetu/impl/kernel/InstanceNorm2d.cc of the reference): per plane the mean, the biased variance and
// (x - mean) / sqrt(var + eps); the gradient is the layer norm's without scale:
// dx = rstd (dy - mean(dy) - xhat mean(dy xhat)).
void InstanceNormCpu(const NDArray& in_arr, NDArray& mean_arr, NDArray& var_arr, NDArray& out_arr, float eps,
                     const Stream& stream) {
  HT_ASSERT_CPU_DEVICE(in_arr);
  HT_ASSERT_SAME_DEVICE(in_arr, mean_arr);
  HT_ASSERT_SAME_DEVICE(in_arr, var_arr);
  HT_ASSERT_SAME_DEVICE(in_arr, out_arr);
  HT_ASSERT_SAME_SHAPE(in_arr, out_arr);
  HT_ASSERT_SAME_DTYPE(in_arr, out_arr);
  HT_ASSERT_SAME_DTYPE(in_arr, mean_arr);
  HT_ASSERT_SAME_DTYPE(in_arr, var_arr);
  HT_ASSERT_CONTIGUOUS(out_arr);
  HT_ASSERT_CONTIGUOUS(mean_arr);
  HT_ASSERT_CONTIGUOUS(var_arr);
  int64_t rows, cols;
  Planes(in_arr, rows, cols);
  HT_ASSERT(int64_t(mean_arr->numel()) == rows && int64_t(var_arr->numel()) == rows)
    << "statistics must hold one value per plane (" << rows << ")";
  if (in_arr->numel() == 0) return;
  HT_DISPATCH_FLOATING_TYPES(in_arr->dtype(), spec_t, "InstanceNormCpu", [&]() {
    cpu::on_stream(stream, "InstanceNormCpu", [=]() {
      NDArray x = Dense(in_arr, stream);
      using A = typename cpu::Arith<spec_t>::type;
      const spec_t* xp = x->data_ptr<spec_t>();
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
          cpu::st<spec_t, A>(yr + i, (cpu::ld<spec_t, A>(xr + i) - mean) * rstd);
        });
      });
    });
  });
}

void InstanceNormGradientCpu(const NDArray& out_grads, const NDArray& in_arr, NDArray& grad_arr,
                             const NDArray& mean_arr, const NDArray& var_arr, float eps, const Stream& stream) {
  HT_ASSERT_CPU_DEVICE(out_grads);
  HT_ASSERT_SAME_DEVICE(out_grads, in_arr);
  HT_ASSERT_SAME_DEVICE(out_grads, grad_arr);
  HT_ASSERT_SAME_DEVICE(out_grads, mean_arr);
  HT_ASSERT_SAME_DEVICE(out_grads, var_arr);
  HT_ASSERT_SAME_SHAPE(out_grads, in_arr);
  HT_ASSERT_SAME_SHAPE(out_grads, grad_arr);
  HT_ASSERT_SAME_DTYPE(out_grads, in_arr);
  HT_ASSERT_SAME_DTYPE(out_grads, grad_arr);
  HT_ASSERT_SAME_DTYPE(out_grads, mean_arr);
  HT_ASSERT_SAME_DTYPE(out_grads, var_arr);
  HT_ASSERT_CONTIGUOUS(grad_arr);
  int64_t rows, cols;
  Planes(in_arr, rows, cols);
  HT_ASSERT(int64_t(mean_arr->numel()) == rows && int64_t(var_arr->numel()) == rows)
    << "statistics must hold one value per plane (" << rows << ")";
  if (in_arr->numel() == 0) return;
  HT_DISPATCH_FLOATING_TYPES(in_arr->dtype(), spec_t, "InstanceNormGradientCpu", [&]() {
    cpu::on_stream(stream, "InstanceNormGradientCpu", [=]() {
      NDArray dy = Dense(out_grads, stream), x = Dense(in_arr, stream);
      NDArray mean = Dense(mean_arr, stream), var = Dense(var_arr, stream);
      using A = typename cpu::Arith<spec_t>::type;
      const spec_t* dyp = dy->data_ptr<spec_t>();
      const spec_t* xp = x->data_ptr<spec_t>();
      const spec_t* mp = mean->data_ptr<spec_t>();
      const spec_t* vp = var->data_ptr<spec_t>();
      spec_t* dxp = grad_arr->data_ptr<spec_t>();
      const A inv = A(1) / A(cols);
      cpu::parallel_rows(rows, cols, [&](int64_t r) {
        const A m = cpu::ld<spec_t, A>(mp + r);
        const A rstd = A(1) / std::sqrt(cpu::ld<spec_t, A>(vp + r) + A(eps));
        const spec_t* dyr = dyp + r * cols;
        const spec_t* xr = xp + r * cols;
        const A s1 = cpu::blocked_sum<A>(cols, [&](int64_t i) { return cpu::ld<spec_t, A>(dyr + i); }) * inv;
        const A s2 = cpu::blocked_sum<A>(cols, [&](int64_t i) {
          return cpu::ld<spec_t, A>(dyr + i) * (cpu::ld<spec_t, A>(xr + i) - m) * rstd;
        }) * inv;
        spec_t* dxr = dxp + r * cols;
        cpu::for_range(0, cols, [&](int64_t i) {
          const A xh = (cpu::ld<spec_t, A>(xr + i) - m) * rstd;
          cpu::st<spec_t, A>(dxr + i, rstd * (cpu::ld<spec_t, A>(dyr + i) - s1 - xh * s2));
        });
      });
    });
  });
}

} // namespace impl
} // namespace hetu
