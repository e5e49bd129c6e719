// LayerNorm / RMSNorm forward kernels for float storage and the double-precision fallback.
#include "hk_norm_fwd_impl.h"

namespace hk {
template int norm_fwd_typed<float>(NormFwdArgs, hipStream_t);

int norm_fwd_f64(const NormFwdArgs& a, hipStream_t s) {
  hipLaunchKernelGGL((norm_fwd_generic_kernel<double, double>), dim3(unsigned(a.n0), unsigned(a.n1), unsigned(a.n2)),
                     dim3(256), 0, s, a);
  return launch_check("norm_fwd_generic_kernel<double>");
}
} // namespace hk
