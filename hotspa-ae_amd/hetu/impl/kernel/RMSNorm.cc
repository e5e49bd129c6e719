// DropoutAddLnFwdCuda / DropoutAddLnBwdCuda and their parallel-residual
// variants: argument lists and checks of hetu/impl/kernel/RMSNorm.cu:91-264,
// :266-470 and :474-826 of the reference (the flash-attention dropout_add_ln
// interface).  The reference leaves the shapes of its outputs to the calling
// op; here every output is checked before a kernel sees it.
#include "hetu/graph/ops/kernel_links.h"
#include "hetu/impl/kernel/kernel_utils.h"
#include "hetu/impl/random/CPURandomState.h"

namespace hetu {
namespace impl {

namespace {

void CheckDense2D(const NDArray& a, DataType dtype, int64_t rows, int64_t cols, const char* name) {
  HT_ASSERT(a.is_defined()) << name << " must be given";
  HT_ASSERT(a->is_cuda()) << name << " must live on the GPU";
  HT_ASSERT(a->is_contiguous()) << name << " must be contiguous";
  HT_ASSERT(a->dtype() == dtype) << name << " must have dtype " << dtype << ", got " << a->dtype();
  HT_ASSERT(a->ndim() == 2 && a->shape(0) == rows && a->shape(1) == cols)
    << name << " must have shape [" << rows << ", " << cols << "], got " << a->shape();
}

void CheckVector(const NDArray& a, DataType dtype, int64_t n, const char* name) {
  HT_ASSERT(a.is_defined()) << name << " must be given";
  HT_ASSERT(a->is_cuda()) << name << " must live on the GPU";
  HT_ASSERT(a->is_contiguous()) << name << " must be contiguous";
  HT_ASSERT(a->dtype() == dtype) << name << " must have dtype " << dtype << ", got " << a->dtype();
  HT_ASSERT(int64_t(a->numel()) == n) << name << " must have " << n << " elements, got " << a->shape();
}

} // namespace

void DropoutAddLnFwdCuda(const NDArray& x0, const NDArray& residual_, const NDArray& gamma, const NDArray& beta_,
                         const NDArray& rowscale_, const NDArray& colscale_, const NDArray& x0_subset_,
                         const NDArray& z_subset_, NDArray& z, NDArray& x, NDArray& dmask, NDArray& mu,
                         NDArray& rsigma, const float dropout_p, const float epsilon, const float rowscale_const,
                         const int64_t z_numrows, bool residual_in_fp32, bool is_rms_norm, const Stream& stream) {
  const auto itype = x0->dtype();
  const auto rtype = residual_.is_defined() ? residual_->dtype() : (residual_in_fp32 ? kFloat32 : x0->dtype());
  const auto wtype = gamma->dtype();

  HT_ASSERT(x0->is_cuda());
  HT_ASSERT(gamma->is_cuda());
  HT_ASSERT(x0->is_contiguous());
  HT_ASSERT(x0->ndim() == 2);
  const bool subset = x0_subset_.is_defined();
  const int64_t rows = subset ? int64_t(x0_subset_->numel()) : x0->shape(0);
  const int64_t cols = x0->shape(1);
  const int64_t x0_rows = x0->shape(0);
  HT_ASSERT(int64_t(gamma->numel()) == cols);
  HT_ASSERT(gamma->is_contiguous());
  if (beta_.is_defined()) CheckVector(beta_, wtype, cols, "beta");
  if (residual_.is_defined()) CheckDense2D(residual_, rtype, rows, cols, "residual");
  if (rowscale_.is_defined()) CheckVector(rowscale_, itype, rows, "rowscale");
  if (colscale_.is_defined()) CheckVector(colscale_, wtype, cols, "colscale");
  if (subset) {
    CheckVector(x0_subset_, kInt32, rows, "x0_subset");
    HT_ASSERT(z_subset_.is_defined()) << "x0_subset comes with z_subset";
    CheckVector(z_subset_, kInt32, rows, "z_subset");
    HT_ASSERT(z_numrows >= 0);
  } else {
    HT_ASSERT(!z_subset_.is_defined()) << "z_subset comes with x0_subset";
  }
  HT_ASSERT((cols % 8 == 0) && (cols <= 8192)) << "hidden size must be a multiple of 8 and at most 8192, got " << cols;
  HT_ASSERT(epsilon >= 0.f);
  HT_ASSERT(dropout_p >= 0.f && dropout_p < 1.f);
  const int64_t z_rows = subset ? z_numrows : rows;
  CheckDense2D(z, itype, z_rows, cols, "z");
  CheckVector(mu, kFloat32, rows, "mu");
  CheckVector(rsigma, kFloat32, rows, "rsigma");
  // the pre-norm sum is kept whenever it differs from x0 in value or dtype (RMSNorm.cu:190)
  const bool save_x = residual_.is_defined() || (dropout_p > 0.f) || rowscale_.is_defined() ||
                      colscale_.is_defined() || subset || (itype != rtype);
  if (save_x) CheckDense2D(x, rtype, rows, cols, "x");
  if (dropout_p > 0.f) CheckDense2D(dmask, kUInt8, x0_rows, cols, "dmask");
  if (rows == 0) return;

  HIPStream hip_stream(stream);
  hip::DeviceGuard guard(hip_stream.device_id());
  hkDropoutAddLnFwdParams p{};
  p.itype = int(itype); p.rtype = int(rtype); p.wtype = int(wtype);
  p.rows = rows; p.cols = cols; p.x0_numrows = x0_rows; p.z_numrows = z_rows;
  p.x0 = x0->raw_data_ptr(); p.residual = PtrOrNull(residual_); p.gamma = gamma->raw_data_ptr();
  p.beta = PtrOrNull(beta_); p.rowscale = PtrOrNull(rowscale_); p.colscale = PtrOrNull(colscale_);
  p.x0_subset = static_cast<const int32_t*>(PtrOrNull(x0_subset_));
  p.z_subset = static_cast<const int32_t*>(PtrOrNull(z_subset_));
  p.z = z->raw_data_ptr(); p.x = save_x ? x->raw_data_ptr() : nullptr;
  p.dmask = dropout_p > 0.f ? static_cast<uint8_t*>(dmask->raw_data_ptr()) : nullptr;
  p.mu = static_cast<float*>(mu->raw_data_ptr()); p.rs = static_cast<float*>(rsigma->raw_data_ptr());
  p.dropout_p = dropout_p; p.epsilon = epsilon; p.rowscale_const = rowscale_const;
  p.is_rms_norm = is_rms_norm ? 1 : 0;
  if (dropout_p > 0.f) p.seed = GenNextRandomSeed();   // RMSNorm.cu:241-250
  HK_CALL(hk_dropout_add_ln_fwd_ex(&p, hip_stream));
  NDArray::MarkUsedBy({x0, residual_, gamma, beta_, rowscale_, colscale_, x0_subset_, z_subset_, z, mu, rsigma},
                      stream);
  if (save_x) NDArray::MarkUsedBy(x, stream);
  if (dropout_p > 0.f) NDArray::MarkUsedBy(dmask, stream);
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
  (void) dgamma_part;
  (void) dbeta_part;
  (void) dcolscale_part;
  const auto itype = dz->dtype();
  const auto rtype = x->dtype();
  const auto wtype = gamma->dtype();

  HT_ASSERT(dropout_p >= 0.f && dropout_p < 1.f);
  if (dropout_p > 0.f) HT_ASSERT(dmask_.is_defined());
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
  const bool subset = x0_subset_.is_defined();
  HT_ASSERT(dz->ndim() == 2);
  HT_ASSERT(dz->shape(1) == cols);
  if (!subset) HT_ASSERT(dz->shape(0) == rows);
  const int64_t z_rows = dz->shape(0);
  const int64_t x0_rows = subset ? x0_numrows : rows;
  HT_ASSERT(int64_t(gamma->numel()) == cols);
  HT_ASSERT(gamma->is_contiguous());
  CheckVector(mu, kFloat32, rows, "mu");
  CheckVector(rsigma, kFloat32, rows, "rsigma");
  if (dx_.is_defined()) CheckDense2D(dx_, rtype, rows, cols, "dx");
  if (dmask_.is_defined()) CheckDense2D(dmask_, kUInt8, x0_rows, cols, "dmask");
  if (rowscale_.is_defined()) CheckVector(rowscale_, itype, rows, "rowscale");
  if (colscale_.is_defined()) {
    CheckVector(colscale_, wtype, cols, "colscale");
    CheckDense2D(x0_, itype, x0_rows, cols, "x0");   // RMSNorm.cu:370-376
    CheckVector(dcolscale, wtype, cols, "dcolscale");
  }
  if (subset) {
    CheckVector(x0_subset_, kInt32, rows, "x0_subset");
    HT_ASSERT(z_subset_.is_defined()) << "x0_subset comes with z_subset";
    CheckVector(z_subset_, kInt32, rows, "z_subset");
    HT_ASSERT(x0_numrows >= 0);
  } else {
    HT_ASSERT(!z_subset_.is_defined()) << "z_subset comes with x0_subset";
  }
  HT_ASSERT((cols % 8 == 0) && (cols <= 8192)) << "hidden size must be a multiple of 8 and at most 8192, got " << cols;
  CheckDense2D(dx0, itype, x0_rows, cols, "dx0");
  CheckVector(dgamma, wtype, cols, "dgamma");
  if (dbeta.is_defined()) CheckVector(dbeta, wtype, cols, "dbeta");
  if (has_residual) CheckDense2D(dresidual, rtype, rows, cols, "dresidual");

  HIPStream hip_stream(stream);
  hip::DeviceGuard guard(hip_stream.device_id());
  hkDropoutAddLnBwdParams p{};
  p.itype = int(itype); p.rtype = int(rtype); p.wtype = int(wtype);
  p.rows = rows; p.cols = cols; p.x0_numrows = x0_rows; p.z_numrows = z_rows;
  p.dz = dz->raw_data_ptr(); p.dx = PtrOrNull(dx_); p.x = x->raw_data_ptr();
  p.x0 = colscale_.is_defined() ? x0_->raw_data_ptr() : nullptr;
  p.dmask = dropout_p > 0.f ? static_cast<const uint8_t*>(dmask_->raw_data_ptr()) : nullptr;
  p.mu = static_cast<const float*>(mu->raw_data_ptr()); p.rs = static_cast<const float*>(rsigma->raw_data_ptr());
  p.gamma = gamma->raw_data_ptr(); p.rowscale = PtrOrNull(rowscale_); p.colscale = PtrOrNull(colscale_);
  p.x0_subset = static_cast<const int32_t*>(PtrOrNull(x0_subset_));
  p.z_subset = static_cast<const int32_t*>(PtrOrNull(z_subset_));
  p.dx0 = dx0->raw_data_ptr(); p.dresidual = has_residual ? dresidual->raw_data_ptr() : nullptr;
  p.dgamma = dgamma->raw_data_ptr(); p.dbeta = MutPtrOrNull(dbeta);
  p.dcolscale = colscale_.is_defined() ? dcolscale->raw_data_ptr() : nullptr;
  p.dropout_p = dropout_p; p.rowscale_const = rowscale_const; p.is_rms_norm = is_rms_norm ? 1 : 0;
  size_t ws_bytes = 0;
  HK_CALL(hk_dropout_add_ln_bwd_ex_workspace_bytes(&p, &ws_bytes));
  NDArray ws = Scratch(ws_bytes, x->device(), stream);
  p.workspace = MutPtrOrNull(ws); p.workspace_bytes = ws_bytes;
  HK_CALL(hk_dropout_add_ln_bwd_ex(&p, hip_stream));
  NDArray::MarkUsedBy({dz, dx_, x, x0_, dmask_, mu, rsigma, gamma, rowscale_, colscale_, x0_subset_, z_subset_,
                       dx0, dgamma, dbeta, dcolscale, ws}, stream);
  if (has_residual) NDArray::MarkUsedBy(dresidual, stream);
}

void DropoutAddLnParallelResidualFwdCuda(const NDArray& x0, const NDArray& x1_, const NDArray& residual_,
                                         const NDArray& gamma0, const NDArray& beta0_, const NDArray& gamma1_,
                                         const NDArray& beta1_, NDArray& z0, NDArray& z1, NDArray& x,
                                         NDArray& dmask0, NDArray& dmask1, NDArray& mu, NDArray& rsigma,
                                         const float dropout_p, const float epsilon, bool residual_in_fp32,
                                         bool is_rms_norm, const Stream& stream) {
  const auto itype = x0->dtype();
  const auto rtype = residual_.is_defined() ? residual_->dtype() : (residual_in_fp32 ? kFloat32 : x0->dtype());
  const auto wtype = gamma0->dtype();

  HT_ASSERT(x0->is_cuda());
  HT_ASSERT(gamma0->is_cuda());
  HT_ASSERT(x0->is_contiguous());
  HT_ASSERT(x0->ndim() == 2);
  const int64_t rows = x0->shape(0), cols = x0->shape(1);
  CheckVector(gamma0, wtype, cols, "gamma0");
  if (x1_.is_defined()) CheckDense2D(x1_, itype, rows, cols, "x1");
  if (residual_.is_defined()) CheckDense2D(residual_, rtype, rows, cols, "residual");
  if (beta0_.is_defined()) CheckVector(beta0_, wtype, cols, "beta0");
  if (gamma1_.is_defined()) CheckVector(gamma1_, wtype, cols, "gamma1");
  if (beta1_.is_defined()) {
    HT_ASSERT(gamma1_.is_defined()) << "beta1 comes with gamma1";
    CheckVector(beta1_, wtype, cols, "beta1");
  }
  HT_ASSERT((cols % 8 == 0) && (cols <= 8192)) << "hidden size must be a multiple of 8 and at most 8192, got " << cols;
  HT_ASSERT(epsilon >= 0.f);
  HT_ASSERT(dropout_p >= 0.f && dropout_p < 1.f);
  CheckDense2D(z0, itype, rows, cols, "z0");
  if (gamma1_.is_defined()) CheckDense2D(z1, itype, rows, cols, "z1");
  CheckVector(mu, kFloat32, rows, "mu");
  CheckVector(rsigma, kFloat32, rows, "rsigma");
  const bool save_x = residual_.is_defined() || x1_.is_defined() || (dropout_p > 0.f) || (itype != rtype);  // :561
  if (save_x) CheckDense2D(x, rtype, rows, cols, "x");
  if (dropout_p > 0.f) {
    CheckDense2D(dmask0, kUInt8, rows, cols, "dmask0");
    if (x1_.is_defined()) CheckDense2D(dmask1, kUInt8, rows, cols, "dmask1");
  }
  if (rows == 0) return;

  HIPStream hip_stream(stream);
  hip::DeviceGuard guard(hip_stream.device_id());
  hkDropoutAddLnFwdParams p{};
  p.itype = int(itype); p.rtype = int(rtype); p.wtype = int(wtype);
  p.rows = rows; p.cols = cols; p.x0_numrows = rows; p.z_numrows = rows;
  p.x0 = x0->raw_data_ptr(); p.x1 = PtrOrNull(x1_); p.residual = PtrOrNull(residual_);
  p.gamma = gamma0->raw_data_ptr(); p.beta = PtrOrNull(beta0_);
  p.gamma1 = PtrOrNull(gamma1_); p.beta1 = PtrOrNull(beta1_);
  p.z = z0->raw_data_ptr(); p.z1 = gamma1_.is_defined() ? z1->raw_data_ptr() : nullptr;
  p.x = save_x ? x->raw_data_ptr() : nullptr;
  if (dropout_p > 0.f) {
    p.dmask = static_cast<uint8_t*>(dmask0->raw_data_ptr());
    if (x1_.is_defined()) p.dmask1 = static_cast<uint8_t*>(dmask1->raw_data_ptr());
    p.seed = GenNextRandomSeed();   // RMSNorm.cu:617-627
  }
  p.mu = static_cast<float*>(mu->raw_data_ptr()); p.rs = static_cast<float*>(rsigma->raw_data_ptr());
  p.dropout_p = dropout_p; p.epsilon = epsilon; p.rowscale_const = 1.f; p.is_rms_norm = is_rms_norm ? 1 : 0;
  HK_CALL(hk_dropout_add_ln_fwd_ex(&p, hip_stream));
  NDArray::MarkUsedBy({x0, x1_, residual_, gamma0, beta0_, gamma1_, beta1_, z0, mu, rsigma}, stream);
  if (gamma1_.is_defined()) NDArray::MarkUsedBy(z1, stream);
  if (save_x) NDArray::MarkUsedBy(x, stream);
  if (dropout_p > 0.f) {
    NDArray::MarkUsedBy(dmask0, stream);
    if (x1_.is_defined()) NDArray::MarkUsedBy(dmask1, stream);
  }
}

void DropoutAddLnParallelResidualBwdCuda(const NDArray& dz0, const NDArray& dz1_, const NDArray& dx_,
                                         const NDArray& x, const NDArray& dmask0_, const NDArray& dmask1_,
                                         const NDArray& mu, const NDArray& rsigma, const NDArray& gamma0,
                                         const NDArray& gamma1_, NDArray& dx0, NDArray& dx1, NDArray& dresidual,
                                         NDArray& dgamma0, NDArray& dbeta0, NDArray& dgamma1, NDArray& dbeta1,
                                         NDArray& dgamma0_part, NDArray& dbeta0_part, NDArray& dgamma1_part,
                                         NDArray& dbeta1_part, const float dropout_p, const bool has_x1,
                                         const bool has_residual, bool is_rms_norm, const Stream& stream) {
  (void) dgamma0_part;
  (void) dbeta0_part;
  (void) dgamma1_part;
  (void) dbeta1_part;
  const auto itype = dz0->dtype();
  const auto rtype = x->dtype();
  const auto wtype = gamma0->dtype();

  HT_ASSERT(dropout_p >= 0.f && dropout_p < 1.f);
  if (dropout_p > 0.f) HT_ASSERT(dmask0_.is_defined());   // RMSNorm.cu:681
  HT_ASSERT(x->is_cuda());
  HT_ASSERT(x->is_contiguous());
  HT_ASSERT(x->ndim() == 2);
  const int64_t rows = x->shape(0), cols = x->shape(1);
  CheckDense2D(dz0, itype, rows, cols, "dz0");
  CheckVector(gamma0, wtype, cols, "gamma0");
  CheckVector(mu, kFloat32, rows, "mu");
  CheckVector(rsigma, kFloat32, rows, "rsigma");
  const bool g1 = gamma1_.is_defined();
  if (g1) {
    CheckVector(gamma1_, wtype, cols, "gamma1");
    CheckDense2D(dz1_, itype, rows, cols, "dz1");
    CheckVector(dgamma1, wtype, cols, "dgamma1");
    CheckVector(dbeta1, wtype, cols, "dbeta1");
  }
  if (dx_.is_defined()) CheckDense2D(dx_, rtype, rows, cols, "dx");
  if (dropout_p > 0.f) {
    CheckDense2D(dmask0_, kUInt8, rows, cols, "dmask0");
    if (has_x1) CheckDense2D(dmask1_, kUInt8, rows, cols, "dmask1");
  }
  HT_ASSERT((cols % 8 == 0) && (cols <= 8192)) << "hidden size must be a multiple of 8 and at most 8192, got " << cols;
  CheckDense2D(dx0, itype, rows, cols, "dx0");
  if (has_x1) CheckDense2D(dx1, itype, rows, cols, "dx1");
  if (has_residual) CheckDense2D(dresidual, rtype, rows, cols, "dresidual");
  CheckVector(dgamma0, wtype, cols, "dgamma0");
  CheckVector(dbeta0, wtype, cols, "dbeta0");

  HIPStream hip_stream(stream);
  hip::DeviceGuard guard(hip_stream.device_id());
  hkDropoutAddLnBwdParams p{};
  p.itype = int(itype); p.rtype = int(rtype); p.wtype = int(wtype);
  p.rows = rows; p.cols = cols; p.x0_numrows = rows; p.z_numrows = rows;
  p.dz = dz0->raw_data_ptr(); p.dz1 = g1 ? dz1_->raw_data_ptr() : nullptr; p.dx = PtrOrNull(dx_);
  p.x = x->raw_data_ptr();
  if (dropout_p > 0.f) {
    p.dmask = static_cast<const uint8_t*>(dmask0_->raw_data_ptr());
    if (has_x1) p.dmask1 = static_cast<const uint8_t*>(dmask1_->raw_data_ptr());
  }
  p.mu = static_cast<const float*>(mu->raw_data_ptr()); p.rs = static_cast<const float*>(rsigma->raw_data_ptr());
  p.gamma = gamma0->raw_data_ptr(); p.gamma1 = PtrOrNull(gamma1_);
  p.dx0 = dx0->raw_data_ptr(); p.dx1 = has_x1 ? dx1->raw_data_ptr() : nullptr;
  p.dresidual = has_residual ? dresidual->raw_data_ptr() : nullptr;
  p.dgamma = dgamma0->raw_data_ptr(); p.dbeta = dbeta0->raw_data_ptr();
  p.dgamma1 = g1 ? dgamma1->raw_data_ptr() : nullptr; p.dbeta1 = g1 ? dbeta1->raw_data_ptr() : nullptr;
  p.dropout_p = dropout_p; p.rowscale_const = 1.f; p.is_rms_norm = is_rms_norm ? 1 : 0;
  size_t ws_bytes = 0;
  HK_CALL(hk_dropout_add_ln_bwd_ex_workspace_bytes(&p, &ws_bytes));
  NDArray ws = Scratch(ws_bytes, x->device(), stream);
  p.workspace = MutPtrOrNull(ws); p.workspace_bytes = ws_bytes;
  HK_CALL(hk_dropout_add_ln_bwd_ex(&p, hip_stream));
  NDArray::MarkUsedBy({dz0, dz1_, dx_, x, dmask0_, dmask1_, mu, rsigma, gamma0, gamma1_, dx0, dgamma0, dbeta0, ws},
                      stream);
  if (has_x1) NDArray::MarkUsedBy(dx1, stream);
  if (has_residual) NDArray::MarkUsedBy(dresidual, stream);
  if (g1) NDArray::MarkUsedBy({dgamma1, dbeta1}, stream);
}

} // namespace impl
} // namespace hetu
