// Operator registration: torch.ops.mi355x.<name> with the schemas of the ATen
// ops the reference implements (its registration goes through PyTorch's
// native_functions.yaml XPU dispatch keys and REGISTER_XPU_DISPATCH,
// src/ATen/native/xpu/LayerNorm.cpp:198-201).  The ops are registered for
// every backend key and reject non-GPU tensors themselves, so a wrong device
// is a clear error instead of a missing-kernel message.  Nothing here touches
// the aten:: namespace; routing aten ops to these kernels is an explicit
// opt-in done from Python.
#include <torch/library.h>

#include "fused_ops.h"
#include "group_norm_ops.h"
#include "norm_ops.h"
#include "softmax_ops.h"

TORCH_LIBRARY(mi355x, m) {
  m.def(
      "native_layer_norm(Tensor input, int[] normalized_shape, Tensor? weight, Tensor? bias, "
      "float eps) -> (Tensor, Tensor, Tensor)",
      &mi355x::native_layer_norm);
  m.def(
      "native_layer_norm_backward(Tensor grad_out, Tensor input, int[] normalized_shape, "
      "Tensor mean, Tensor rstd, Tensor? weight, Tensor? bias, bool[3] output_mask) -> "
      "(Tensor, Tensor, Tensor)",
      &mi355x::native_layer_norm_backward);
  m.def(
      "_fused_rms_norm(Tensor input, int[] normalized_shape, Tensor? weight, float? eps) -> "
      "(Tensor, Tensor)",
      &mi355x::_fused_rms_norm);
  m.def(
      "_fused_rms_norm_backward(Tensor grad_out, Tensor input, int[] normalized_shape, "
      "Tensor rstd, Tensor? weight, bool[2] output_mask) -> (Tensor, Tensor)",
      &mi355x::_fused_rms_norm_backward);
  m.def("_softmax(Tensor self, int dim, bool half_to_float) -> Tensor", &mi355x::_softmax);
  m.def("_log_softmax(Tensor self, int dim, bool half_to_float) -> Tensor",
        &mi355x::_log_softmax);
  m.def("_softmax.out(Tensor self, int dim, bool half_to_float, *, Tensor(a!) out) -> Tensor(a!)",
        &mi355x::_softmax_out);
  m.def(
      "_log_softmax.out(Tensor self, int dim, bool half_to_float, *, Tensor(a!) out) -> "
      "Tensor(a!)",
      &mi355x::_log_softmax_out);
  m.def(
      "_softmax_backward_data(Tensor grad_output, Tensor output, int dim, ScalarType "
      "input_dtype) -> Tensor",
      &mi355x::_softmax_backward_data);
  m.def(
      "_log_softmax_backward_data(Tensor grad_output, Tensor output, int dim, ScalarType "
      "input_dtype) -> Tensor",
      &mi355x::_log_softmax_backward_data);
  m.def(
      "_softmax_backward_data.out(Tensor grad_output, Tensor output, int dim, ScalarType "
      "input_dtype, *, Tensor(a!) grad_input) -> Tensor(a!)",
      &mi355x::_softmax_backward_data_out);
  m.def(
      "_log_softmax_backward_data.out(Tensor grad_output, Tensor output, int dim, ScalarType "
      "input_dtype, *, Tensor(a!) out) -> Tensor(a!)",
      &mi355x::_log_softmax_backward_data_out);
  m.def("_safe_softmax(Tensor self, int dim, ScalarType? dtype=None) -> Tensor",
        &mi355x::_safe_softmax);
  m.def(
      "_masked_softmax(Tensor self, Tensor mask, int? dim=None, int? mask_type=None) -> Tensor",
      &mi355x::_masked_softmax);
  m.def(
      "_masked_softmax_backward(Tensor grad_output, Tensor output, Tensor mask, int? dim=None) "
      "-> Tensor",
      &mi355x::_masked_softmax_backward);
  m.def(
      "native_group_norm(Tensor input, Tensor? weight, Tensor? bias, int N, int C, int HxW, "
      "int group, float eps) -> (Tensor, Tensor, Tensor)",
      &mi355x::native_group_norm);
  m.def(
      "native_group_norm_backward(Tensor grad_out, Tensor input, Tensor mean, Tensor rstd, "
      "Tensor? weight, int N, int C, int HxW, int group, bool[3] output_mask) -> "
      "(Tensor, Tensor, Tensor)",
      &mi355x::native_group_norm_backward);
  // fused residual add -> norm (-> cast): new operator surface, not aten ops
  m.def(
      "add_layer_norm(Tensor input, Tensor residual, int[] normalized_shape, Tensor? weight, "
      "Tensor? bias, float eps, ScalarType? out_dtype=None) -> (Tensor, Tensor, Tensor, Tensor)",
      &mi355x::add_layer_norm);
  m.def(
      "add_layer_norm_(Tensor input, Tensor(a!) residual, int[] normalized_shape, Tensor? weight, "
      "Tensor? bias, float eps, ScalarType? out_dtype=None) -> (Tensor, Tensor, Tensor)",
      &mi355x::add_layer_norm_);
  m.def(
      "add_layer_norm_backward(Tensor grad_y, Tensor? grad_h, Tensor h, int[] normalized_shape, "
      "Tensor mean, Tensor rstd, Tensor? weight, Tensor? bias, bool[3] output_mask) -> "
      "(Tensor, Tensor, Tensor)",
      &mi355x::add_layer_norm_backward);
  m.def(
      "add_rms_norm(Tensor input, Tensor residual, int[] normalized_shape, Tensor? weight, "
      "float? eps, ScalarType? out_dtype=None) -> (Tensor, Tensor, Tensor)",
      &mi355x::add_rms_norm);
  m.def(
      "add_rms_norm_(Tensor input, Tensor(a!) residual, int[] normalized_shape, Tensor? weight, "
      "float? eps, ScalarType? out_dtype=None) -> (Tensor, Tensor)",
      &mi355x::add_rms_norm_);
  m.def(
      "add_rms_norm_backward(Tensor grad_y, Tensor? grad_h, Tensor h, int[] normalized_shape, "
      "Tensor rstd, Tensor? weight, bool[2] output_mask) -> (Tensor, Tensor)",
      &mi355x::add_rms_norm_backward);
  m.def("install_group_norm_dispatch_stubs() -> ()", &mi355x::install_group_norm_dispatch_stubs);
  m.def("install_layer_norm_dispatch_stubs() -> ()", &mi355x::install_layer_norm_dispatch_stubs);
  m.def("uninstall_group_norm_dispatch_stubs() -> ()",
        &mi355x::uninstall_group_norm_dispatch_stubs);
  m.def("uninstall_layer_norm_dispatch_stubs() -> ()",
        &mi355x::uninstall_layer_norm_dispatch_stubs);
}
