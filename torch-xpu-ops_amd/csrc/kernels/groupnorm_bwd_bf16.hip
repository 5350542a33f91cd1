// GroupNorm backward kernels, bf16 rows, bf16 weights.
#include "groupnorm_launch.hpp"
namespace rownorm {
template int launch_group_norm_bwd<bf16, bf16>(const Plan&, const GroupNormBwdArgs&, hipStream_t);
}  // namespace rownorm
