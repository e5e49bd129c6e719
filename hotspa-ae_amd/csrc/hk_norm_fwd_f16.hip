// LayerNorm / RMSNorm forward kernels for fp16 storage.
#include "hk_norm_fwd_impl.h"

namespace hk {
template int norm_fwd_typed<fp16>(NormFwdArgs, hipStream_t);
} // namespace hk
