// GroupNorm backward kernels, fp32 rows, fp32 weights.
#include "groupnorm_launch.hpp"
namespace rownorm {
template int launch_group_norm_bwd<float, float>(const Plan&, const GroupNormBwdArgs&, hipStream_t);
}  // namespace rownorm
