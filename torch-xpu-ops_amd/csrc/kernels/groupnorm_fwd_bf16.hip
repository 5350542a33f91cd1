// GroupNorm forward kernels, bf16 rows, bf16 weights.
#include "groupnorm_launch.hpp"
namespace rownorm {
template int launch_group_norm_fwd<bf16, bf16>(const Plan&, const GroupNormFwdArgs&, hipStream_t);
}  // namespace rownorm
