// ATen-signature softmax / log_softmax operators backed by the MI355X kernels.
#pragma once
#include <ATen/ATen.h>

namespace mi355x {

// Kernel-entry level: same parameter lists as the reference's
// src/ATen/native/xpu/sycl/SoftMaxKernels.h:19-43.
void _softmax_kernel(const at::Tensor& input, int64_t dim, bool half_to_float,
                     const at::Tensor& output);
void _log_softmax_kernel(const at::Tensor& input, int64_t dim, bool half_to_float,
                         const at::Tensor& output);
void _softmax_backward_kernel(const at::Tensor& grad, const at::Tensor& output, int64_t dim,
                              bool half_to_float, const at::Tensor& grad_input);
void _log_softmax_backward_kernel(const at::Tensor& grad, const at::Tensor& output, int64_t dim,
                                  bool half_to_float, const at::Tensor& grad_input);

// SoftMaxKernels.h:45-58.
at::Tensor _safe_softmax_kernel(const at::Tensor& self, int64_t dim, bool half_to_float);
at::Tensor masked_softmax_kernel(const at::Tensor& input, const at::Tensor& mask,
                                 std::optional<int64_t> dim, std::optional<int64_t> mask_type);
at::Tensor masked_softmax_backward_kernel(const at::Tensor& grad, const at::Tensor& output,
                                          const at::Tensor& mask, std::optional<int64_t> dim);

// Operator level: the functional and out= forms of the structured ops the
// reference implements in src/ATen/native/xpu/SoftMax.cpp:22-100.
at::Tensor _softmax(const at::Tensor& self, int64_t dim, bool half_to_float);
at::Tensor _log_softmax(const at::Tensor& self, int64_t dim, bool half_to_float);
at::Tensor& _softmax_out(const at::Tensor& self, int64_t dim, bool half_to_float, at::Tensor& out);
at::Tensor& _log_softmax_out(const at::Tensor& self, int64_t dim, bool half_to_float,
                             at::Tensor& out);
at::Tensor _softmax_backward_data(const at::Tensor& grad_output, const at::Tensor& output,
                                  int64_t dim, at::ScalarType input_dtype);
at::Tensor _log_softmax_backward_data(const at::Tensor& grad_output, const at::Tensor& output,
                                      int64_t dim, at::ScalarType input_dtype);
at::Tensor& _softmax_backward_data_out(const at::Tensor& grad_output, const at::Tensor& output,
                                       int64_t dim, at::ScalarType input_dtype,
                                       at::Tensor& grad_input);
at::Tensor& _log_softmax_backward_data_out(const at::Tensor& grad_output, const at::Tensor& output,
                                           int64_t dim, at::ScalarType input_dtype,
                                           at::Tensor& grad_input);

// _safe_softmax_xpu, masked_softmax_xpu, masked_softmax_backward_xpu
// (src/ATen/native/xpu/SoftMax.cpp:102-126).
at::Tensor _safe_softmax(const at::Tensor& self, int64_t dim,
                         std::optional<at::ScalarType> dtype);
at::Tensor _masked_softmax(const at::Tensor& self, const at::Tensor& mask,
                           std::optional<int64_t> dim, std::optional<int64_t> mask_type);
at::Tensor _masked_softmax_backward(const at::Tensor& grad_output, const at::Tensor& output,
                                    const at::Tensor& mask, std::optional<int64_t> dim);

}  // namespace mi355x
