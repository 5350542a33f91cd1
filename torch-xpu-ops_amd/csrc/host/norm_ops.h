// ATen-signature LayerNorm / RMSNorm operators backed by the MI355X kernels.
#pragma once
#include <ATen/ATen.h>
#include <array>
#include <optional>
#include <tuple>

namespace mi355x {

// Kernel-entry level: same parameter lists as the reference's
// src/ATen/native/xpu/sycl/LayerNormKernels.h:19-59.
void layer_norm_kernel(const at::Tensor& X, const at::Tensor& gamma, const at::Tensor& beta,
                       int64_t M, int64_t N, double eps, at::Tensor* Y, at::Tensor* mean,
                       at::Tensor* rstd);
void layer_norm_backward_kernel(const at::Tensor& dY, const at::Tensor& X, const at::Tensor& mean,
                                const at::Tensor& rstd, const at::Tensor& gamma, int64_t M,
                                int64_t N, at::Tensor* dX, at::Tensor* dgamma, at::Tensor* dbeta);
void rms_norm_kernel(const at::Tensor& X, const at::Tensor& gamma, int64_t M, int64_t N,
                     double eps, at::Tensor* Y, at::Tensor* rstd);
void rms_norm_backward_kernel(const at::Tensor& dY, const at::Tensor& X, const at::Tensor& rstd,
                              const at::Tensor& gamma, int64_t M, int64_t N, at::Tensor* dX,
                              at::Tensor* dgamma);

// Operator level: same signatures as src/ATen/native/xpu/LayerNorm.cpp:35-40,
// 99-107, 203-207, 255-261 in the reference.
std::tuple<at::Tensor, at::Tensor, at::Tensor> native_layer_norm(
    const at::Tensor& input, at::IntArrayRef normalized_shape,
    const std::optional<at::Tensor>& weight_opt, const std::optional<at::Tensor>& bias_opt,
    double epsilon);
std::tuple<at::Tensor, at::Tensor, at::Tensor> native_layer_norm_backward(
    const at::Tensor& grad_output, const at::Tensor& input, at::IntArrayRef normalized_shape,
    const at::Tensor& mean, const at::Tensor& rstd, const std::optional<at::Tensor>& weight_opt,
    const std::optional<at::Tensor>& bias_opt, std::array<bool, 3> grad_input_mask);
std::tuple<at::Tensor, at::Tensor> _fused_rms_norm(const at::Tensor& input,
                                                   at::IntArrayRef normalized_shape,
                                                   const std::optional<at::Tensor>& weight_opt,
                                                   std::optional<double> eps_opt);
std::tuple<at::Tensor, at::Tensor> _fused_rms_norm_backward(
    const at::Tensor& dY, const at::Tensor& input, at::IntArrayRef normalized_shape,
    const at::Tensor& rstd, const std::optional<at::Tensor>& weight_opt,
    std::array<bool, 2> grad_input_mask);

// Points ATen's own LayerNormKernel / LayerNormBackwardKernel dispatch stubs at
// the kernels above for GPU tensors (what REGISTER_XPU_DISPATCH does at load
// time in LayerNorm.cpp:198-201 of the reference).  Explicit, never at import.
// ATen callers that go through the stubs (nested-tensor layer_norm is one) then
// run these kernels; float64 calls are passed on to the kernels that were
// registered before.  uninstall_* puts the previous kernels back.  Not
// synchronized with concurrent calls of the ops: install at start-up.
void install_layer_norm_dispatch_stubs();
void uninstall_layer_norm_dispatch_stubs();

}  // namespace mi355x
