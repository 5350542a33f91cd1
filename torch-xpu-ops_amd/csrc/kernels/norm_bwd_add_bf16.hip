// LayerNorm / RMSNorm bwd kernels that add the gradient of the residual path to dx, rows bf16,
// weights bf16.
#include "norm_launch.hpp"
namespace rownorm {
template int launch_norm_bwd<bf16, bf16, false, true>(const Plan&, const NormBwdArgs&, hipStream_t);
template int launch_norm_bwd<bf16, bf16, true, true>(const Plan&, const NormBwdArgs&, hipStream_t);
}  // namespace rownorm
