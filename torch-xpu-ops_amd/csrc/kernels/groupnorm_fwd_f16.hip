// GroupNorm forward kernels, fp16 rows, fp16 weights.
#include "groupnorm_launch.hpp"
namespace rownorm {
template int launch_group_norm_fwd<f16, f16>(const Plan&, const GroupNormFwdArgs&, hipStream_t);
}  // namespace rownorm
