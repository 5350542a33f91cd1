// GroupNorm backward kernels, fp16 rows, fp32 weights.
#include "groupnorm_launch.hpp"
namespace rownorm {
template int launch_group_norm_bwd<f16, float>(const Plan&, const GroupNormBwdArgs&, hipStream_t);
}  // namespace rownorm
