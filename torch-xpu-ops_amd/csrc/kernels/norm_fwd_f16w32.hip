// LayerNorm / RMSNorm fwd kernels, rows f16, weights float.
#include "norm_launch.hpp"
namespace rownorm {
template int launch_norm_fwd<f16, float, false>(const Plan&, const NormFwdArgs&, hipStream_t);
template int launch_norm_fwd<f16, float, true>(const Plan&, const NormFwdArgs&, hipStream_t);
}  // namespace rownorm
