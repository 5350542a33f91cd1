// ATen-signature GroupNorm operators backed by the MI355X kernels.
#pragma once
#include <ATen/ATen.h>
#include <array>
#include <optional>
#include <tuple>

namespace mi355x {

// Kernel-entry level: same parameter lists as the reference's
// src/ATen/native/xpu/sycl/GroupNormKernels.h:17-42 (ATen's forward_fn /
// backward_fn of ATen/native/group_norm.h).
void group_norm_kernel(const at::Tensor& X, const at::Tensor& gamma, const at::Tensor& beta,
                       int64_t N, int64_t C, int64_t HxW, int64_t group, double eps, at::Tensor& Y,
                       at::Tensor& mean, at::Tensor& rstd);
void group_norm_backward_kernel(const at::Tensor& dY, const at::Tensor& X, const at::Tensor& mean,
                                const at::Tensor& rstd, const at::Tensor& gamma, int64_t N,
                                int64_t C, int64_t HxW, int64_t group, at::Tensor& dX,
                                at::Tensor& dgamma, at::Tensor& dbeta);

// Operator level: aten::native_group_norm / native_group_norm_backward, the
// host functions that sit above the kernel entries (upstream ATen code in the
// reference's build; its own part is the dispatch registration in
// src/ATen/native/xpu/GroupNorm.cpp:19-23).
std::tuple<at::Tensor, at::Tensor, at::Tensor> native_group_norm(
    const at::Tensor& input, const std::optional<at::Tensor>& weight_opt,
    const std::optional<at::Tensor>& bias_opt, int64_t N, int64_t C, int64_t HxW, int64_t group,
    double eps);
std::tuple<at::Tensor, at::Tensor, at::Tensor> native_group_norm_backward(
    const at::Tensor& grad_out, const at::Tensor& input, const at::Tensor& mean,
    const at::Tensor& rstd, const std::optional<at::Tensor>& weight_opt, int64_t N, int64_t C,
    int64_t HxW, int64_t group, std::array<bool, 3> output_mask);

// Points ATen's GroupNormKernel / GroupNormBackwardKernel dispatch stubs at the
// kernel entries above for GPU tensors: REGISTER_XPU_DISPATCH in
// GroupNorm.cpp:19-23 of the reference.  Explicit, never at import.  ATen's own
// native_group_norm host function then reaches these kernels; float64 calls are
// passed on to the kernels that were registered before.  uninstall_* puts the
// previous kernels back.  Not synchronized with concurrent calls of the ops.
void install_group_norm_dispatch_stubs();
void uninstall_group_norm_dispatch_stubs();

}  // namespace mi355x
