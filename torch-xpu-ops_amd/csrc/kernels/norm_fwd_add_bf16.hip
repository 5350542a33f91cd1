// LayerNorm / RMSNorm fwd kernels with the residual add fused in (h = x + res is written and
// normalized), rows bf16, weights bf16.
#include "norm_launch.hpp"
namespace rownorm {
template int launch_norm_fwd<bf16, bf16, false, bf16, true>(const Plan&, const NormFwdArgs&, hipStream_t);
template int launch_norm_fwd<bf16, bf16, true, bf16, true>(const Plan&, const NormFwdArgs&, hipStream_t);
}  // namespace rownorm
