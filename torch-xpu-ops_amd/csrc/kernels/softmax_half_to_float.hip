// half_to_float softmax variants: fp16 rows in / fp32 out (forward) and fp32
// grads in / fp16 input-gradient out (backward), the pair the reference allows
// in SoftMaxKernels.cpp:2131-2135 and src/ATen/native/xpu/SoftMax.cpp:49-55.
#include "softmax_launch.hpp"
namespace rownorm {
template int launch_softmax_fwd<f16, float>(const Plan&, const SoftmaxFwdArgs&, hipStream_t);
template int launch_softmax_bwd<float, f16>(const Plan&, const SoftmaxBwdArgs&, hipStream_t);
}  // namespace rownorm
