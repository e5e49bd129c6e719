// BatchNormCuda / BatchNormGradientCuda: arguments and meaning of
// hetu/impl/kernel/BatchNorm.cu:8-83 and :84-165 of the reference, which hands the
// work to cuDNN's spatial batch normalisation in training mode.  save_var holds
// what cuDNN saves there: the inverse standard deviation 1 / sqrt(var + eps).
// Scale, bias and every statistic are float32 for float16 / bfloat16 data.
#include "hetu/graph/ops/kernel_links.h"
#include "hetu/impl/kernel/kernel_utils.h"
#include "hetu/impl/utils/cpu_utils.h"
#include "hetu/impl/utils/dispatch.h"

#include <cmath>

namespace hetu {
namespace impl {

namespace {
DataType ParamType(DataType data) {
  return (data == kFloat16 || data == kBFloat16) ? kFloat32 : data;
}

void CheckParam(const NDArray& a, const NDArray& data, DataType dtype, int64_t channels, const char* name) {
  HT_ASSERT(a.is_defined()) << name << " must be given";
  HT_ASSERT(a->device() == data->device()) << name << " must live on " << data->device() << ", got " << a->device();
  HT_ASSERT(a->dtype() == dtype) << name << " must have dtype " << dtype << ", got " << a->dtype();
  HT_ASSERT(int64_t(a->numel()) == channels) << name << " must have one value per channel (" << channels
                                             << "), got " << a->shape();
  HT_ASSERT(a->is_contiguous()) << name << " must be contiguous";
}

void SplitNCHW(const NDArray& x, int64_t& N, int64_t& C, int64_t& HW) {
  HT_ASSERT(x->ndim() >= 2) << "Batch normalisation needs [N, C, ...], got " << x->shape();
  N = x->shape(0);
  C = x->shape(1);
  HW = 1;
  for (size_t i = 2; i < x->ndim(); ++i) HW *= x->shape(int64_t(i));
}
} // namespace

void BatchNormCuda(const NDArray& input_X, const NDArray& bn_scale, const NDArray& bn_bias, NDArray& output_Y,
                   double momentum, double eps, NDArray& running_mean, NDArray& running_var, NDArray& save_mean,
                   NDArray& save_var, const Stream& stream) {
  HT_ASSERT_CUDA_DEVICE(input_X);
  HT_ASSERT_SAME_DEVICE(input_X, output_Y);
  HT_ASSERT_SAME_SHAPE(input_X, output_Y);
  HT_ASSERT_SAME_DTYPE(input_X, output_Y);
  HT_ASSERT_CONTIGUOUS(output_Y);
  int64_t N, C, HW;
  SplitNCHW(input_X, N, C, HW);
  const DataType pt = ParamType(input_X->dtype());
  CheckParam(bn_scale, input_X, pt, C, "bn_scale");
  CheckParam(bn_bias, input_X, pt, C, "bn_bias");
  CheckParam(running_mean, input_X, pt, C, "running_mean");
  CheckParam(running_var, input_X, pt, C, "running_var");
  CheckParam(save_mean, input_X, pt, C, "save_mean");
  CheckParam(save_var, input_X, pt, C, "save_var");
  if (input_X->numel() == 0) return;

  HIPStream hip_stream(stream);
  hip::DeviceGuard guard(hip_stream.device_id());
  NDArray x = Dense(input_X, stream);
  size_t ws_bytes = 0;
  HK_CALL(hk_batch_norm_workspace_bytes(int(x->dtype()), N, C, HW, &ws_bytes));
  NDArray ws = Scratch(ws_bytes, x->device(), stream);
  HK_CALL(hk_batch_norm_fwd(int(x->dtype()), x->raw_data_ptr(), bn_scale->raw_data_ptr(), bn_bias->raw_data_ptr(),
                            output_Y->raw_data_ptr(), momentum, eps, running_mean->raw_data_ptr(),
                            running_var->raw_data_ptr(), save_mean->raw_data_ptr(), save_var->raw_data_ptr(), N, C,
                            HW, MutPtrOrNull(ws), ws_bytes, hip_stream));
  NDArray::MarkUsedBy({x, bn_scale, bn_bias, output_Y, running_mean, running_var, save_mean, save_var, ws}, stream);
}

void BatchNormGradientCuda(const NDArray& gradient_Y, const NDArray& input_X, const NDArray& bn_scale,
                           NDArray& gradient_X, NDArray& gradient_bn_scale, NDArray& gradient_bn_bias, double eps,
                           NDArray& save_mean, NDArray& save_var, const Stream& stream) {
  (void) eps;   // already inside the saved inverse standard deviation
  HT_ASSERT_CUDA_DEVICE(gradient_Y);
  HT_ASSERT_SAME_DEVICE(gradient_Y, input_X);
  HT_ASSERT_SAME_DEVICE(gradient_Y, gradient_X);
  HT_ASSERT_SAME_SHAPE(gradient_Y, input_X);
  HT_ASSERT_SAME_SHAPE(gradient_X, input_X);
  HT_ASSERT_SAME_DTYPE(gradient_Y, input_X);
  HT_ASSERT_SAME_DTYPE(gradient_X, input_X);
  HT_ASSERT_CONTIGUOUS(gradient_X);
  int64_t N, C, HW;
  SplitNCHW(input_X, N, C, HW);
  const DataType pt = ParamType(input_X->dtype());
  CheckParam(bn_scale, input_X, pt, C, "bn_scale");
  CheckParam(gradient_bn_scale, input_X, pt, C, "gradient_bn_scale");
  CheckParam(gradient_bn_bias, input_X, pt, C, "gradient_bn_bias");
  CheckParam(save_mean, input_X, pt, C, "save_mean");
  CheckParam(save_var, input_X, pt, C, "save_var");
  if (input_X->numel() == 0) return;

  HIPStream hip_stream(stream);
  hip::DeviceGuard guard(hip_stream.device_id());
  NDArray x = Dense(input_X, stream), dy = Dense(gradient_Y, stream);
  size_t ws_bytes = 0;
  HK_CALL(hk_batch_norm_workspace_bytes(int(x->dtype()), N, C, HW, &ws_bytes));
  NDArray ws = Scratch(ws_bytes, x->device(), stream);
  HK_CALL(hk_batch_norm_bwd(int(x->dtype()), dy->raw_data_ptr(), x->raw_data_ptr(), bn_scale->raw_data_ptr(),
                            gradient_X->raw_data_ptr(), gradient_bn_scale->raw_data_ptr(),
                            gradient_bn_bias->raw_data_ptr(), save_mean->raw_data_ptr(), save_var->raw_data_ptr(), N,
                            C, HW, MutPtrOrNull(ws), ws_bytes, hip_stream));
  NDArray::MarkUsedBy({dy, x, bn_scale, gradient_X, gradient_bn_scale, gradient_bn_bias, save_mean, save_var, ws},
                      stream);
}

// Host twins (hetu/impl/kernel/BatchNorm.cc of the reference, a oneDNN primitive there) with the accelerator
// path's conventions, so that a graph can move between the two: save_var holds 1 / sqrt(var + eps), the running
// variance takes the unbiased estimate, parameters and statistics are float32 for 16-bit data.  One channel at a
// time: mean, then the centred sum of squares, then the output.
void BatchNormCpu(const NDArray& input_X, const NDArray& bn_scale, const NDArray& bn_bias, NDArray& output_Y,
                  double momentum, double eps, NDArray& running_mean, NDArray& running_var, NDArray& save_mean,
                  NDArray& save_var, const Stream& stream) {
  HT_ASSERT_CPU_DEVICE(input_X);
  HT_ASSERT_SAME_DEVICE(input_X, output_Y);
  HT_ASSERT_SAME_SHAPE(input_X, output_Y);
  HT_ASSERT_SAME_DTYPE(input_X, output_Y);
  HT_ASSERT_CONTIGUOUS(output_Y);
  int64_t N, C, HW;
  SplitNCHW(input_X, N, C, HW);
  const DataType pt = ParamType(input_X->dtype());
  CheckParam(bn_scale, input_X, pt, C, "bn_scale");
  CheckParam(bn_bias, input_X, pt, C, "bn_bias");
  CheckParam(running_mean, input_X, pt, C, "running_mean");
  CheckParam(running_var, input_X, pt, C, "running_var");
  CheckParam(save_mean, input_X, pt, C, "save_mean");
  CheckParam(save_var, input_X, pt, C, "save_var");
  if (input_X->numel() == 0) return;
  HT_DISPATCH_FLOATING_TYPES(input_X->dtype(), spec_t, "BatchNormCpu", [&]() {
    cpu::on_stream(stream, "BatchNormCpu", [=]() {
      NDArray x = Dense(input_X, stream);
      using A = typename cpu::Arith<spec_t>::type;   // also the parameters' storage type
      const spec_t* xp = x->data_ptr<spec_t>();
      spec_t* yp = output_Y->data_ptr<spec_t>();
      const A* scale = bn_scale->data_ptr<A>();
      const A* bias = bn_bias->data_ptr<A>();
      A* rm = running_mean->data_ptr<A>();
      A* rv = running_var->data_ptr<A>();
      A* sm = save_mean->data_ptr<A>();
      A* sv = save_var->data_ptr<A>();
      const int64_t m = N * HW;
      cpu::parallel_rows(C, m, [&](int64_t c) {
        A sum = A(0);
        for (int64_t n = 0; n < N; ++n) {
          const spec_t* plane = xp + (n * C + c) * HW;
          sum += cpu::blocked_sum<A>(HW, [&](int64_t i) { return cpu::ld<spec_t, A>(plane + i); });
        }
        const A mean = sum / A(m);
        A sq = A(0);
        for (int64_t n = 0; n < N; ++n) {
          const spec_t* plane = xp + (n * C + c) * HW;
          sq += cpu::blocked_sum<A>(HW, [&](int64_t i) {
            const A d = cpu::ld<spec_t, A>(plane + i) - mean;
            return d * d;
          });
        }
        const A var = sq / A(m);
        const A invstd = A(1) / std::sqrt(var + A(eps));
        const A unbiased = m > 1 ? sq / A(m - 1) : var;
        sm[c] = mean;
        sv[c] = invstd;
        rm[c] = A((1.0 - momentum) * double(rm[c]) + momentum * double(mean));
        rv[c] = A((1.0 - momentum) * double(rv[c]) + momentum * double(unbiased));
        const A w = invstd * scale[c], b = bias[c];
        for (int64_t n = 0; n < N; ++n) {
          const spec_t* plane = xp + (n * C + c) * HW;
          spec_t* out = yp + (n * C + c) * HW;
          cpu::for_range(0, HW, [&](int64_t i) {
            cpu::st<spec_t, A>(out + i, (cpu::ld<spec_t, A>(plane + i) - mean) * w + b);
          });
        }
      });
    });
  });
}

void BatchNormGradientCpu(const NDArray& gradient_Y, const NDArray& input_X, const NDArray& bn_scale,
                          NDArray& gradient_X, NDArray& gradient_bn_scale, NDArray& gradient_bn_bias, double eps,
                          NDArray& save_mean, NDArray& save_var, const Stream& stream) {
  (void) eps;   // already inside the saved inverse standard deviation
  HT_ASSERT_CPU_DEVICE(gradient_Y);
  HT_ASSERT_SAME_DEVICE(gradient_Y, input_X);
  HT_ASSERT_SAME_DEVICE(gradient_Y, gradient_X);
  HT_ASSERT_SAME_SHAPE(gradient_Y, input_X);
  HT_ASSERT_SAME_SHAPE(gradient_X, input_X);
  HT_ASSERT_SAME_DTYPE(gradient_Y, input_X);
  HT_ASSERT_SAME_DTYPE(gradient_X, input_X);
  HT_ASSERT_CONTIGUOUS(gradient_X);
  int64_t N, C, HW;
  SplitNCHW(input_X, N, C, HW);
  const DataType pt = ParamType(input_X->dtype());
  CheckParam(bn_scale, input_X, pt, C, "bn_scale");
  CheckParam(gradient_bn_scale, input_X, pt, C, "gradient_bn_scale");
  CheckParam(gradient_bn_bias, input_X, pt, C, "gradient_bn_bias");
  CheckParam(save_mean, input_X, pt, C, "save_mean");
  CheckParam(save_var, input_X, pt, C, "save_var");
  if (input_X->numel() == 0) return;
  HT_DISPATCH_FLOATING_TYPES(input_X->dtype(), spec_t, "BatchNormGradientCpu", [&]() {
    cpu::on_stream(stream, "BatchNormGradientCpu", [=]() {
      NDArray x = Dense(input_X, stream), dy = Dense(gradient_Y, stream);
      using A = typename cpu::Arith<spec_t>::type;
      const spec_t* xp = x->data_ptr<spec_t>();
      const spec_t* dyp = dy->data_ptr<spec_t>();
      spec_t* dxp = gradient_X->data_ptr<spec_t>();
      const A* scale = bn_scale->data_ptr<A>();
      const A* sm = save_mean->data_ptr<A>();
      const A* sv = save_var->data_ptr<A>();
      A* dscale = gradient_bn_scale->data_ptr<A>();
      A* dbias = gradient_bn_bias->data_ptr<A>();
      const int64_t m = N * HW;
      cpu::parallel_rows(C, m, [&](int64_t c) {
        const A mean = sm[c], invstd = sv[c];
        A sum_dy = A(0), sum_dy_xhat = A(0);
        for (int64_t n = 0; n < N; ++n) {
          const spec_t* xr = xp + (n * C + c) * HW;
          const spec_t* dr = dyp + (n * C + c) * HW;
          sum_dy += cpu::blocked_sum<A>(HW, [&](int64_t i) { return cpu::ld<spec_t, A>(dr + i); });
          sum_dy_xhat += cpu::blocked_sum<A>(HW, [&](int64_t i) {
            return cpu::ld<spec_t, A>(dr + i) * (cpu::ld<spec_t, A>(xr + i) - mean) * invstd;
          });
        }
        dscale[c] = sum_dy_xhat;
        dbias[c] = sum_dy;
        const A w = scale[c] * invstd, k1 = sum_dy / A(m), k2 = sum_dy_xhat / A(m);
        for (int64_t n = 0; n < N; ++n) {
          const spec_t* xr = xp + (n * C + c) * HW;
          const spec_t* dr = dyp + (n * C + c) * HW;
          spec_t* out = dxp + (n * C + c) * HW;
          cpu::for_range(0, HW, [&](int64_t i) {
            const A xh = (cpu::ld<spec_t, A>(xr + i) - mean) * invstd;
            cpu::st<spec_t, A>(out + i, w * (cpu::ld<spec_t, A>(dr + i) - k1 - xh * k2));
          });
        }
      });
    });
  });
}

} // namespace impl
} // namespace hetu
