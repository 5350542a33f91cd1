// Non-innermost-dimension softmax / log_softmax kernels, fp16 in / fp32 out forward, fp32 grads / fp16 input gradient backward.
#include "softmax_strided_launch.hpp"
namespace rownorm {
template int launch_softmax_strided_fwd<f16, float>(const StridedPlan&, const SoftmaxStridedFwdArgs&,
                                                hipStream_t);
template int launch_softmax_strided_bwd<float, f16>(const StridedPlan&, const SoftmaxStridedBwdArgs&,
                                                hipStream_t);
}  // namespace rownorm
