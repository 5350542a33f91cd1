// LayerNorm / RMSNorm fwd kernels, rows float, weights float, y written as f16.
#include "norm_launch.hpp"
namespace rownorm {
template int launch_norm_fwd<float, float, false, f16, false>(const Plan&, const NormFwdArgs&, hipStream_t);
template int launch_norm_fwd<float, float, true, f16, false>(const Plan&, const NormFwdArgs&, hipStream_t);
}  // namespace rownorm
