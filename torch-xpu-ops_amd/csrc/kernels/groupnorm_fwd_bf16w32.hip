// GroupNorm forward kernels, bf16 rows, fp32 weights.
#include "groupnorm_launch.hpp"
namespace rownorm {
template int launch_group_norm_fwd<bf16, float>(const Plan&, const GroupNormFwdArgs&, hipStream_t);
}  // namespace rownorm
