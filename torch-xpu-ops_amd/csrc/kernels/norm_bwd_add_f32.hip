// LayerNorm / RMSNorm bwd kernels that add the gradient of the residual path to dx, rows float,
// weights float.
#include "norm_launch.hpp"
namespace rownorm {
template int launch_norm_bwd<float, float, false, true>(const Plan&, const NormBwdArgs&, hipStream_t);
template int launch_norm_bwd<float, float, true, true>(const Plan&, const NormBwdArgs&, hipStream_t);
}  // namespace rownorm
