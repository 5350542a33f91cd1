// Non-innermost-dimension softmax / log_softmax kernels, fp32 in, fp32 out.
#include "softmax_strided_launch.hpp"
namespace rownorm {
template int launch_softmax_strided_fwd<float, float>(const StridedPlan&, const SoftmaxStridedFwdArgs&,
                                                hipStream_t);
template int launch_softmax_strided_bwd<float, float>(const StridedPlan&, const SoftmaxStridedBwdArgs&,
                                                hipStream_t);
}  // namespace rownorm
