// LayerNorm / RMSNorm bwd kernels, rows float, weights float.
#include "norm_launch.hpp"
namespace rownorm {
template int launch_norm_bwd<float, float, false>(const Plan&, const NormBwdArgs&, hipStream_t);
template int launch_norm_bwd<float, float, true>(const Plan&, const NormBwdArgs&, hipStream_t);
}  // namespace rownorm
