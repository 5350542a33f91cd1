// LayerNorm / RMSNorm fwd kernels, rows float, weights float.
#include "norm_launch.hpp"
namespace rownorm {
template int launch_norm_fwd<float, float, false>(const Plan&, const NormFwdArgs&, hipStream_t);
template int launch_norm_fwd<float, float, true>(const Plan&, const NormFwdArgs&, hipStream_t);
}  // namespace rownorm
