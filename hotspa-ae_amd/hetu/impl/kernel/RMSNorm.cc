// DropoutAddLnFwdCuda / DropoutAddLnBwdCuda: argument list and checks of
// hetu/impl/kernel/RMSNorm.cu:91-264 and :266-470 of the reference (the
// flash-attention dropout_add_ln interface), for the configuration Hetu's
// RMSNorm and LayerNorm modules call it with: no dropout, no row / column
// scaling, no row subsets.  Any of those raises not_implemented instead of
// silently computing something else.
#include "hetu/graph/ops/kernel_links.h"
#include "hetu/impl/kernel/kernel_utils.h"

namespace hetu {
namespace impl {

void DropoutAddLnFwdCuda(const NDArray& x0, const NDArray& residual_, const NDArray& gamma, const NDArray& beta_,
                         const NDArray& rowscale_, const NDArray& colscale_, const NDArray& x0_subset_,
                         const NDArray& z_subset_, NDArray& z, NDArray& x, NDArray& dmask, NDArray& mu,
                         NDArray& rsigma, const float dropout_p, const float epsilon, const float rowscale_const,
                         const int64_t z_numrows, bool residual_in_fp32, bool is_rms_norm, const Stream& stream) {
  (void) dmask;
  (void) z_numrows;
  const auto itype = x0->dtype();
  const auto rtype = residual_.is_defined() ? residual_->dtype() : (residual_in_fp32 ? kFloat32 : x0->dtype());
  const auto wtype = gamma->dtype();

  HT_ASSERT(x0->is_cuda());
  HT_ASSERT(gamma->is_cuda());
  HT_ASSERT(x0->is_contiguous());
  HT_ASSERT(x0->ndim() == 2);
  const int64_t rows = x0->shape(0), cols = x0->shape(1);
  HT_ASSERT(int64_t(gamma->numel()) == cols);
  HT_ASSERT(gamma->is_contiguous());
  if (beta_.is_defined()) {
    HT_ASSERT(beta_->dtype() == wtype);
    HT_ASSERT(beta_->is_cuda());
    HT_ASSERT(beta_->is_contiguous());
    HT_ASSERT(beta_->shape() == gamma->shape());
  }
  if (residual_.is_defined()) {
    HT_ASSERT(residual_->is_cuda());
    HT_ASSERT(residual_->is_contiguous());
    HT_ASSERT(residual_->shape() == x0->shape());
  }
  HT_NOT_IMPLEMENTED_IF(dropout_p != 0.f) << "dropout inside the fused norm (p = " << dropout_p << ")";
  HT_NOT_IMPLEMENTED_IF(rowscale_.is_defined() || colscale_.is_defined() || rowscale_const != 1.f)
    << "row / column scaling inside the fused norm";
  HT_NOT_IMPLEMENTED_IF(x0_subset_.is_defined() || z_subset_.is_defined()) << "row subsets inside the fused norm";
  HT_ASSERT((cols % 8 == 0) && (cols <= 8192)) << "hidden size must be a multiple of 8 and at most 8192, got " << cols;
  HT_ASSERT(epsilon >= 0.f);
  HT_ASSERT(z.is_defined() && z->dtype() == itype && z->shape() == x0->shape() && z->is_contiguous());
  HT_ASSERT(mu.is_defined() && mu->dtype() == kFloat32 && int64_t(mu->numel()) == rows && mu->is_contiguous());
  HT_ASSERT(rsigma.is_defined() && rsigma->dtype() == kFloat32 && int64_t(rsigma->numel()) == rows &&
            rsigma->is_contiguous());
  // the pre-norm sum is kept when it differs from x0 in value or dtype
  const bool save_x = residual_.is_defined() || (itype != rtype);
  if (save_x) {
    HT_ASSERT(x.is_defined() && x->dtype() == rtype && x->shape() == x0->shape() && x->is_contiguous())
      << "x must be given (dtype " << rtype << ") when a residual is added or the residual dtype differs";
  }
  if (rows == 0) return;

  HIPStream hip_stream(stream);
  hip::DeviceGuard guard(hip_stream.device_id());
  HK_CALL(hk_dropout_add_ln_fwd(int(itype), int(rtype), int(wtype), x0->raw_data_ptr(), PtrOrNull(residual_),
                                gamma->raw_data_ptr(), PtrOrNull(beta_), z->raw_data_ptr(),
                                save_x ? x->raw_data_ptr() : nullptr, mu->raw_data_ptr(), rsigma->raw_data_ptr(),
                                rows, cols, epsilon, is_rms_norm ? 1 : 0, hip_stream));
  NDArray::MarkUsedBy({x0, residual_, gamma, beta_, z, mu, rsigma}, stream);
  if (save_x) NDArray::MarkUsedBy(x, stream);
}

void DropoutAddLnBwdCuda(const NDArray& dz, const NDArray& dx_, const NDArray& x, const NDArray& x0_,
                         const NDArray& dmask_, const NDArray& mu, const NDArray& rsigma, const NDArray& gamma,
                         const NDArray& rowscale_, const NDArray& colscale_, const NDArray& x0_subset_,
                         const NDArray& z_subset_, NDArray& dx0, NDArray& dresidual, NDArray& dgamma,
                         NDArray& dbeta, NDArray& dgamma_part, NDArray& dbeta_part, NDArray& dcolscale,
                         NDArray& dcolscale_part, const float dropout_p, const float rowscale_const,
                         const int64_t x0_numrows, const bool has_residual, bool is_rms_norm,
                         const Stream& stream) {
  // The per-block partial sums live in pool scratch sized by the kernel's own
  // plan; caller-provided part buffers are accepted and left untouched.
  (void) x0_;
  (void) dmask_;
  (void) dgamma_part;
  (void) dbeta_part;
  (void) dcolscale;
  (void) dcolscale_part;
  (void) x0_numrows;
  const auto itype = dz->dtype();
  const auto rtype = x->dtype();
  const auto wtype = gamma->dtype();

  HT_ASSERT(mu->dtype() == kFloat32);
  HT_ASSERT(rsigma->dtype() == kFloat32);
  HT_ASSERT(x->is_cuda());
  HT_ASSERT(dz->is_cuda());
  HT_ASSERT(mu->is_cuda());
  HT_ASSERT(rsigma->is_cuda());
  HT_ASSERT(gamma->is_cuda());
  HT_ASSERT(x->is_contiguous());
  HT_ASSERT(dz->is_contiguous());
  HT_ASSERT(x->ndim() == 2);
  const int64_t rows = x->shape(0), cols = x->shape(1);
  HT_ASSERT(dz->ndim() == 2);
  HT_ASSERT(dz->shape(0) == rows && dz->shape(1) == cols);
  HT_ASSERT(int64_t(gamma->numel()) == cols);
  HT_ASSERT(gamma->is_contiguous());
  HT_ASSERT(int64_t(mu->numel()) == rows && mu->is_contiguous());
  HT_ASSERT(int64_t(rsigma->numel()) == rows && rsigma->is_contiguous());
  if (dx_.is_defined()) {
    HT_ASSERT(dx_->dtype() == rtype);
    HT_ASSERT(dx_->is_cuda());
    HT_ASSERT(dx_->is_contiguous());
    HT_ASSERT(dx_->shape() == x->shape());
  }
  HT_NOT_IMPLEMENTED_IF(dropout_p != 0.f) << "dropout inside the fused norm (p = " << dropout_p << ")";
  HT_NOT_IMPLEMENTED_IF(rowscale_.is_defined() || colscale_.is_defined() || rowscale_const != 1.f)
    << "row / column scaling inside the fused norm";
  HT_NOT_IMPLEMENTED_IF(x0_subset_.is_defined() || z_subset_.is_defined()) << "row subsets inside the fused norm";
  HT_ASSERT((cols % 8 == 0) && (cols <= 8192)) << "hidden size must be a multiple of 8 and at most 8192, got " << cols;
  HT_ASSERT(dx0.is_defined() && dx0->dtype() == itype && dx0->shape() == x->shape() && dx0->is_contiguous());
  HT_ASSERT(dgamma.is_defined() && dgamma->dtype() == wtype && int64_t(dgamma->numel()) == cols &&
            dgamma->is_contiguous());
  if (dbeta.is_defined())
    HT_ASSERT(dbeta->dtype() == wtype && int64_t(dbeta->numel()) == cols && dbeta->is_contiguous());
  if (has_residual) {
    HT_ASSERT(dresidual.is_defined() && dresidual->dtype() == rtype && dresidual->shape() == x->shape() &&
              dresidual->is_contiguous())
      << "dresidual must be given (dtype " << rtype << ") when the forward added a residual";
  }

  HIPStream hip_stream(stream);
  hip::DeviceGuard guard(hip_stream.device_id());
  if (rows == 0) {
    const size_t bytes = size_t(cols) * DataType2Size(wtype);
    HK_CALL(hk_memset(dgamma->raw_data_ptr(), 0, bytes, hip_stream));
    if (dbeta.is_defined()) HK_CALL(hk_memset(dbeta->raw_data_ptr(), 0, bytes, hip_stream));
    NDArray::MarkUsedBy({dgamma, dbeta}, stream);
    return;
  }
  size_t ws_bytes = 0;
  HK_CALL(hk_norm_bwd_workspace_bytes(int(itype), rows, cols, &ws_bytes));
  NDArray ws = Scratch(ws_bytes, x->device(), stream);
  HK_CALL(hk_dropout_add_ln_bwd(int(itype), int(rtype), int(wtype), dz->raw_data_ptr(), PtrOrNull(dx_),
                                x->raw_data_ptr(), mu->raw_data_ptr(), rsigma->raw_data_ptr(),
                                gamma->raw_data_ptr(), dx0->raw_data_ptr(),
                                has_residual ? dresidual->raw_data_ptr() : nullptr, dgamma->raw_data_ptr(),
                                MutPtrOrNull(dbeta), rows, cols, is_rms_norm ? 1 : 0, MutPtrOrNull(ws), ws_bytes,
                                hip_stream));
  NDArray::MarkUsedBy({dz, dx_, x, mu, rsigma, gamma, dx0, dgamma, dbeta, ws}, stream);
  if (has_residual) NDArray::MarkUsedBy(dresidual, stream);
}

} // namespace impl
} // namespace hetu
