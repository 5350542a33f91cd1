// LayerNorm / RMSNorm fwd kernels with the residual add fused in (h = x + res is written and
// normalized), rows f16, weights f16.
#include "norm_launch.hpp"
namespace rownorm {
template int launch_norm_fwd<f16, f16, false, f16, true>(const Plan&, const NormFwdArgs&, hipStream_t);
template int launch_norm_fwd<f16, f16, true, f16, true>(const Plan&, const NormFwdArgs&, hipStream_t);
}  // namespace rownorm
