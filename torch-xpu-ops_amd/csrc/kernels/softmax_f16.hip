// softmax / log_softmax forward and backward kernels, f16 in, f16 out.
#include "softmax_launch.hpp"
namespace rownorm {
template int launch_softmax_fwd<f16, f16>(const Plan&, const SoftmaxFwdArgs&, hipStream_t);
template int launch_softmax_bwd<f16, f16>(const Plan&, const SoftmaxBwdArgs&, hipStream_t);
}  // namespace rownorm
