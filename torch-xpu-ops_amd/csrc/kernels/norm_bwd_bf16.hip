// LayerNorm / RMSNorm bwd kernels, rows bf16, weights bf16.
#include "norm_launch.hpp"
namespace rownorm {
template int launch_norm_bwd<bf16, bf16, false>(const Plan&, const NormBwdArgs&, hipStream_t);
template int launch_norm_bwd<bf16, bf16, true>(const Plan&, const NormBwdArgs&, hipStream_t);
}  // namespace rownorm
