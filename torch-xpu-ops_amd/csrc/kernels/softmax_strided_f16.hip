// Non-innermost-dimension softmax / log_softmax kernels, fp16 in, fp16 out.
#include "softmax_strided_launch.hpp"
namespace rownorm {
template int launch_softmax_strided_fwd<f16, f16>(const StridedPlan&, const SoftmaxStridedFwdArgs&,
                                                hipStream_t);
template int launch_softmax_strided_bwd<f16, f16>(const StridedPlan&, const SoftmaxStridedBwdArgs&,
                                                hipStream_t);
}  // namespace rownorm
