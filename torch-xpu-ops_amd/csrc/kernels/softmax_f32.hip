// softmax / log_softmax forward and backward kernels, float in, float out.
#include "softmax_launch.hpp"
namespace rownorm {
template int launch_softmax_fwd<float, float>(const Plan&, const SoftmaxFwdArgs&, hipStream_t);
template int launch_softmax_bwd<float, float>(const Plan&, const SoftmaxBwdArgs&, hipStream_t);
}  // namespace rownorm
