// LayerNorm / RMSNorm backward kernels for float storage and the double-precision fallback.
#include "hk_norm_bwd_impl.h"

namespace hk {
template BwdPlan plan_norm_bwd<float>(int64_t, int, bool);
template int norm_bwd_typed<float>(NormBwdArgs, int, void*, void*, void*, size_t, hipStream_t);

int norm_bwd_f64(const NormBwdArgs& a, int mode, void* dgamma, void* dbeta, hipStream_t s) {
  hipLaunchKernelGGL((norm_bwd_generic_dx_kernel<double, double>), dim3(unsigned(a.n0), unsigned(a.n1), unsigned(a.n2)),
                     dim3(256), 0, s, a, mode);
  int rc = launch_check("norm_bwd_generic_dx_kernel<double>");
  if (rc != HK_OK) return rc;
  if (dgamma || dbeta) {
    hipLaunchKernelGGL((norm_bwd_generic_cols_kernel<double, double>), dim3(unsigned((a.cols + 63) / 64)),
                       dim3(256), 0, s, a, mode, static_cast<double*>(dgamma), static_cast<double*>(dbeta));
    rc = launch_check("norm_bwd_generic_cols_kernel<double>");
  }
  return rc;
}
} // namespace hk
