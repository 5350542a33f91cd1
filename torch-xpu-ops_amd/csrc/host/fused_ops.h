// Fused residual add -> LayerNorm / RMSNorm (-> output cast) operators backed by the MI355X
// kernels: the step either side of the norm in a transformer block.  The reference has no such
// operators (its forward, src/ATen/native/xpu/sycl/LayerNormKernels.cpp:469-586, starts from the
// summed row); the results equal its norm applied to `input + residual` rounded to the row dtype.
#pragma once
#include <ATen/ATen.h>
#include <array>
#include <optional>
#include <tuple>

namespace mi355x {

// -> (y, h, mean, rstd): h = input + residual (same dtype and shape), y = layer_norm(h) in
// out_dtype (the input dtype, or Half / BFloat16 for a float32 input), mean / rstd float32 shaped
// like native_layer_norm's.
std::tuple<at::Tensor, at::Tensor, at::Tensor, at::Tensor> add_layer_norm(
    const at::Tensor& input, const at::Tensor& residual, at::IntArrayRef normalized_shape,
    const std::optional<at::Tensor>& weight_opt, const std::optional<at::Tensor>& bias_opt,
    double eps, std::optional<at::ScalarType> out_dtype);

// The in-place form: h is written into `residual` (the usual update of the residual stream, no
// third tensor).  -> (y, mean, rstd)
std::tuple<at::Tensor, at::Tensor, at::Tensor> add_layer_norm_(
    const at::Tensor& input, at::Tensor& residual, at::IntArrayRef normalized_shape,
    const std::optional<at::Tensor>& weight_opt, const std::optional<at::Tensor>& bias_opt,
    double eps, std::optional<at::ScalarType> out_dtype);

// -> (dh, dweight, dbias): dh = layer_norm backward of grad_y at h, plus grad_h when given; it
// is the gradient of both `input` and `residual`.
std::tuple<at::Tensor, at::Tensor, at::Tensor> add_layer_norm_backward(
    const at::Tensor& grad_y, const std::optional<at::Tensor>& grad_h_opt, const at::Tensor& h,
    at::IntArrayRef normalized_shape, const at::Tensor& mean, const at::Tensor& rstd,
    const std::optional<at::Tensor>& weight_opt, const std::optional<at::Tensor>& bias_opt,
    std::array<bool, 3> output_mask);

// -> (y, h, rstd)
std::tuple<at::Tensor, at::Tensor, at::Tensor> add_rms_norm(
    const at::Tensor& input, const at::Tensor& residual, at::IntArrayRef normalized_shape,
    const std::optional<at::Tensor>& weight_opt, std::optional<double> eps_opt,
    std::optional<at::ScalarType> out_dtype);

// In place on `residual`.  -> (y, rstd)
std::tuple<at::Tensor, at::Tensor> add_rms_norm_(
    const at::Tensor& input, at::Tensor& residual, at::IntArrayRef normalized_shape,
    const std::optional<at::Tensor>& weight_opt, std::optional<double> eps_opt,
    std::optional<at::ScalarType> out_dtype);

// -> (dh, dweight)
std::tuple<at::Tensor, at::Tensor> add_rms_norm_backward(
    const at::Tensor& grad_y, const std::optional<at::Tensor>& grad_h_opt, const at::Tensor& h,
    at::IntArrayRef normalized_shape, const at::Tensor& rstd,
    const std::optional<at::Tensor>& weight_opt, std::array<bool, 2> output_mask);

}  // namespace mi355x
