// LayerNorm / RMSNorm fwd kernels, rows float, weights float, y written as f16 (residual add fused in).
#include "norm_launch.hpp"
namespace rownorm {
template int launch_norm_fwd<float, float, false, f16, true>(const Plan&, const NormFwdArgs&, hipStream_t);
template int launch_norm_fwd<float, float, true, f16, true>(const Plan&, const NormFwdArgs&, hipStream_t);
}  // namespace rownorm
