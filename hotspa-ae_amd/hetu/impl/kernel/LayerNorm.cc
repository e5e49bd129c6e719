// LayerNormCuda / LayerNormGradientCuda: same arguments and meaning as
// hetu/impl/kernel/LayerNorm.cu:66-121 and :235-337 of the reference (statistics
// are mean and VARIANCE, stored in the data dtype), run by the gfx950 kernels
// behind hk_layer_norm_fwd / hk_layer_norm_bwd.  The operator takes non-contiguous
// arrays (hetu/graph/ops/LayerNorm.h:78-80): row-pitched inputs and outputs go to
// the kernels as they are, any other input layout through a dense copy.
#include "hetu/graph/ops/kernel_links.h"
#include "hetu/impl/kernel/kernel_utils.h"

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
  int64_t x_pitch = cols, y_pitch = cols;
  HT_ASSERT_ROW_PITCHED(out_arr, reduce_dims, &y_pitch);
  HT_ASSERT(int64_t(ln_scale->numel()) == cols && int64_t(ln_bias->numel()) == cols)
    << "scale " << ln_scale->shape() << " / bias " << ln_bias->shape() << " do not match " << cols << " columns";
  HT_ASSERT(int64_t(mean_arr->numel()) == rows && int64_t(var_arr->numel()) == rows)
    << "statistics must hold one value per row (" << rows << ")";
  if (in_arr->numel() == 0) return;

  HIPStream hip_stream(stream);
  hip::DeviceGuard guard(hip_stream.device_id());
  NDArray x = RowOperand(in_arr, reduce_dims, stream, &x_pitch);
  NDArray g = Dense(ln_scale, stream), b = Dense(ln_bias, stream);
  const int dt = int(in_arr->dtype());
  HK_CALL(hk_layer_norm_fwd_pitched(dt, x->raw_data_ptr(), x_pitch, g->raw_data_ptr(), b->raw_data_ptr(),
                                    out_arr->raw_data_ptr(), y_pitch, mean_arr->raw_data_ptr(),
                                    var_arr->raw_data_ptr(), dt, HK_STAT_VAR, rows, cols, eps, hip_stream));
  NDArray::MarkUsedBy({x, g, b, mean_arr, var_arr, out_arr}, stream);
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
  int64_t dy_pitch = cols, x_pitch = cols, dx_pitch = cols;
  HT_ASSERT_ROW_PITCHED(grad_arr, reduce_dims, &dx_pitch);
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
  NDArray dy = RowOperand(out_grads, reduce_dims, stream, &dy_pitch);
  NDArray x = RowOperand(in_arr, reduce_dims, stream, &x_pitch), g = Dense(ln_scale, stream);
  NDArray mean = Dense(mean_arr, stream), var = Dense(var_arr, stream);
  size_t ws_bytes = 0;
  HK_CALL(hk_norm_bwd_workspace_bytes(dt, rows, cols, &ws_bytes));
  NDArray ws = Scratch(ws_bytes, in_arr->device(), stream);
  HK_CALL(hk_layer_norm_bwd_pitched(dt, dy->raw_data_ptr(), dy_pitch, x->raw_data_ptr(), x_pitch, g->raw_data_ptr(),
                                    /*beta=*/nullptr, mean->raw_data_ptr(), var->raw_data_ptr(), dt, HK_STAT_VAR,
                                    grad_arr->raw_data_ptr(), dx_pitch, grad_scale->raw_data_ptr(),
                                    grad_bias->raw_data_ptr(), rows, cols, eps, /*memory_efficient=*/0,
                                    /*clamp_gamma=*/0, MutPtrOrNull(ws), ws_bytes, hip_stream));
  NDArray::MarkUsedBy({dy, x, g, mean, var, grad_arr, grad_scale, grad_bias, ws}, stream);
}

void LayerNormCpu(const NDArray&, const NDArray&, const NDArray&, NDArray&, NDArray&, NDArray&, int64_t, float,
                  const Stream&) {
  HT_NOT_IMPLEMENTED << "LayerNorm has no host kernel in this build (the reference's is a oneDNN primitive); "
                        "move the arrays to the accelerator";
}

void LayerNormGradientCpu(const NDArray&, const NDArray&, const NDArray&, NDArray&, NDArray&, NDArray&,
                          const NDArray&, const NDArray&, int64_t, float, const Stream&) {
  HT_NOT_IMPLEMENTED << "LayerNormGradient has no host kernel in this build; move the arrays to the accelerator";
}

} // namespace impl
} // namespace hetu
