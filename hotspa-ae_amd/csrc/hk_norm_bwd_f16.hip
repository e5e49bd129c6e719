// LayerNorm / RMSNorm backward kernels for fp16 storage.
#include "hk_norm_bwd_impl.h"

namespace hk {
template BwdPlan plan_norm_bwd<fp16>(int64_t, int, bool);
template int norm_bwd_typed<fp16>(NormBwdArgs, int, void*, void*, void*, size_t, hipStream_t);
} // namespace hk
