// LayerNorm / RMSNorm bwd kernels, rows f16, weights f16.
#include "norm_launch.hpp"
namespace rownorm {
template int launch_norm_bwd<f16, f16, false>(const Plan&, const NormBwdArgs&, hipStream_t);
template int launch_norm_bwd<f16, f16, true>(const Plan&, const NormBwdArgs&, hipStream_t);
}  // namespace rownorm
