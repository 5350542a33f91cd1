// LayerNorm / RMSNorm fwd kernels with the residual add fused in (h = x + res is written and
// normalized), rows float, weights float.
#include "norm_launch.hpp"
namespace rownorm {
template int launch_norm_fwd<float, float, false, float, true>(const Plan&, const NormFwdArgs&, hipStream_t);
template int launch_norm_fwd<float, float, true, float, true>(const Plan&, const NormFwdArgs&, hipStream_t);
}  // namespace rownorm
