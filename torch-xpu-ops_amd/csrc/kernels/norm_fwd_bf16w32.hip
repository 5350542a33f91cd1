// LayerNorm / RMSNorm fwd kernels, rows bf16, weights float.
#include "norm_launch.hpp"
namespace rownorm {
template int launch_norm_fwd<bf16, float, false>(const Plan&, const NormFwdArgs&, hipStream_t);
template int launch_norm_fwd<bf16, float, true>(const Plan&, const NormFwdArgs&, hipStream_t);
}  // namespace rownorm
