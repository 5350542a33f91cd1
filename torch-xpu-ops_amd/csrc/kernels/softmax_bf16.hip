// softmax / log_softmax forward and backward kernels, bf16 in, bf16 out.
#include "softmax_launch.hpp"
namespace rownorm {
template int launch_softmax_fwd<bf16, bf16>(const Plan&, const SoftmaxFwdArgs&, hipStream_t);
template int launch_softmax_bwd<bf16, bf16>(const Plan&, const SoftmaxBwdArgs&, hipStream_t);
}  // namespace rownorm
