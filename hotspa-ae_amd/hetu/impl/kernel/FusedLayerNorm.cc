// FusedLayerNormCuda / FusedLayerNormGradientCuda: arguments and meaning of
// hetu/impl/kernel/FusedLayerNorm.cu:967-1004 and :1006-1144 of the reference
// (statistics are mean and 1/sqrt(var+eps) in fp32; `inplace` = the
// memory-efficient backward that gets the forward OUTPUT instead of the input).
#include "hetu/graph/ops/kernel_links.h"
#include "hetu/impl/kernel/kernel_utils.h"

namespace hetu {
namespace impl {

void FusedLayerNormCuda(const NDArray& in_arr, const NDArray& ln_scale, const NDArray& ln_bias, NDArray& mean_arr,
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
  HT_ASSERT(mean_arr->dtype() == kFloat32 && var_arr->dtype() == kFloat32)
    << "the fused layer norm keeps its statistics in float32, got " << mean_arr->dtype() << " / "
    << var_arr->dtype();
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
  // row-pitched arrays and views with permuted leading dimensions are read and written in place
  RowPlan plan(reduce_dims, stream);
  RowPlan::Slot& x = plan.Input(in_arr);
  RowPlan::Slot& y = plan.Output(out_arr);
  plan.Resolve();
  NDArray g = Dense(ln_scale, stream), b = Dense(ln_bias, stream);
  HK_CALL(hk_layer_norm_fwd_strided_rows(int(in_arr->dtype()), x.ptr(), x.steps, g->raw_data_ptr(),
                                         b->raw_data_ptr(), y.ptr(), y.steps, mean_arr->raw_data_ptr(),
                                         var_arr->raw_data_ptr(), HK_FLOAT32, HK_STAT_RSTD, plan.level_rows(), cols,
                                         eps, hip_stream));
  NDArray::MarkUsedBy({x.array, g, b, mean_arr, var_arr, y.array}, stream);
  plan.Commit();
}

void FusedLayerNormGradientCuda(const NDArray& out_grads, const NDArray& in_arr, const NDArray& ln_scale,
                                const NDArray& ln_bias, NDArray& grad_arr, NDArray& grad_scale, NDArray& grad_bias,
                                const NDArray& mean_arr, const NDArray& var_arr, int64_t reduce_dims, float eps,
                                bool inplace, const Stream& stream) {
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
  HT_ASSERT(mean_arr->dtype() == kFloat32 && var_arr->dtype() == kFloat32)
    << "the fused layer norm keeps its statistics in float32";
  HT_ASSERT(!inplace || ln_bias.is_defined()) << "the memory-efficient backward needs the bias to undo it";
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
  RowPlan::Slot& xy = plan.Input(in_arr);
  RowPlan::Slot& dx = plan.Output(grad_arr);
  plan.Resolve();
  NDArray g = Dense(ln_scale, stream);
  NDArray b = Dense(ln_bias, stream), mean = Dense(mean_arr, stream), rstd = Dense(var_arr, stream);
  size_t ws_bytes = 0;
  HK_CALL(hk_norm_bwd_workspace_bytes(dt, rows, cols, &ws_bytes));
  NDArray ws = Scratch(ws_bytes, in_arr->device(), stream);
  // gamma enters dx through clamp_by_magnitude(gamma, eps) in both modes
  // (FusedLayerNorm.cu:911-938)
  HK_CALL(hk_layer_norm_bwd_strided_rows(dt, dy.ptr(), dy.steps, xy.ptr(), xy.steps, g->raw_data_ptr(), PtrOrNull(b),
                                         mean->raw_data_ptr(), rstd->raw_data_ptr(), HK_FLOAT32, HK_STAT_RSTD,
                                         dx.ptr(), dx.steps, grad_scale->raw_data_ptr(), grad_bias->raw_data_ptr(),
                                         plan.level_rows(), cols, eps, inplace ? 1 : 0, /*clamp_gamma=*/1,
                                         MutPtrOrNull(ws), ws_bytes, hip_stream));
  NDArray::MarkUsedBy({dy.array, xy.array, g, b, mean, rstd, dx.array, grad_scale, grad_bias, ws}, stream);
  plan.Commit();
}

} // namespace impl
} // namespace hetu
