// LayerNorm / RMSNorm forward kernels for bf16 storage.
#include "hk_norm_fwd_impl.h"

namespace hk {
template int norm_fwd_typed<bf16>(NormFwdArgs, hipStream_t);
} // namespace hk
