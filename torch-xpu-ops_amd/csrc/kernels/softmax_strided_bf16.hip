// Non-innermost-dimension softmax / log_softmax kernels, bf16 in, bf16 out.
#include "softmax_strided_launch.hpp"
namespace rownorm {
template int launch_softmax_strided_fwd<bf16, bf16>(const StridedPlan&, const SoftmaxStridedFwdArgs&,
                                                hipStream_t);
template int launch_softmax_strided_bwd<bf16, bf16>(const StridedPlan&, const SoftmaxStridedBwdArgs&,
                                                hipStream_t);
}  // namespace rownorm
