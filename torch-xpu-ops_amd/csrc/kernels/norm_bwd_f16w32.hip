// LayerNorm / RMSNorm bwd kernels, rows f16, weights float.
#include "norm_launch.hpp"
namespace rownorm {
template int launch_norm_bwd<f16, float, false>(const Plan&, const NormBwdArgs&, hipStream_t);
template int launch_norm_bwd<f16, float, true>(const Plan&, const NormBwdArgs&, hipStream_t);
}  // namespace rownorm
