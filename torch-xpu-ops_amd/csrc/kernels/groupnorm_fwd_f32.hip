// GroupNorm forward kernels, fp32 rows, fp32 weights.
#include "groupnorm_launch.hpp"
namespace rownorm {
template int launch_group_norm_fwd<float, float>(const Plan&, const GroupNormFwdArgs&, hipStream_t);
}  // namespace rownorm
