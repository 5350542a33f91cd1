// softmax / log_softmax host operators.  Contracts follow the reference's
// src/ATen/native/xpu/SoftMax.cpp:22-100 and the host_softmax /
// host_softmax_backward entry code in SoftMaxKernels.cpp:2125-2276.
//
// The kernels reduce over the innermost dimension of a dense tensor.  A
// reduction over another dimension is served by moving that dimension last
// (one transposing copy in, one out) rather than by a separate strided kernel.
#include "softmax_ops.h"

#include <ATen/WrapDimUtils.h>
#include <ATen/native/Resize.h>

#include "host_common.h"

namespace mi355x {
namespace {

using at::Tensor;

// Forward on dense [rows, N] data where `dim` is already innermost.
void forward_lastdim(const Tensor& in, const Tensor& out, bool is_log, const char* op) {
  const int64_t N = in.dim() == 0 ? 1 : in.size(-1);
  const int64_t rows = N == 0 ? 0 : in.numel() / N;
  check_status(mi355x_softmax_fwd(in.const_data_ptr(), out.mutable_data_ptr(), rows, N,
                                  to_rownorm_dtype(in.scalar_type(), op),
                                  to_rownorm_dtype(out.scalar_type(), op), is_log ? 1 : 0,
                                  current_stream(in)),
               op);
}

void backward_lastdim(const Tensor& grad, const Tensor& y, const Tensor& gi, bool is_log,
                      const char* op) {
  const int64_t N = y.dim() == 0 ? 1 : y.size(-1);
  const int64_t rows = N == 0 ? 0 : y.numel() / N;
  check_status(mi355x_softmax_bwd(grad.const_data_ptr(), y.const_data_ptr(),
                                  gi.mutable_data_ptr(), rows, N,
                                  to_rownorm_dtype(grad.scalar_type(), op),
                                  to_rownorm_dtype(gi.scalar_type(), op), is_log ? 1 : 0,
                                  current_stream(y)),
               op);
}

// host_softmax, SoftMaxKernels.cpp:2125-2178: half_to_float needs a Half
// input (:2131-2135); 0-dim tensors are viewed as [1] (:2143-2144); an empty
// tensor is a no-op (:2150).
void softmax_forward_entry(const Tensor& input_, int64_t dim_, bool half_to_float,
                           const Tensor& output, bool is_log, const char* op) {
  check_gpu(input_, op, "input");
  check_same_device(input_, output, op, "output");
  if (half_to_float) {
    TORCH_CHECK(input_.scalar_type() == at::kHalf, op,
                ": conversion is supported for Half type only");
  }
  const at::ScalarType want = half_to_float ? at::kFloat : input_.scalar_type();
  TORCH_CHECK(output.scalar_type() == want, op, ": output dtype ", output.scalar_type(),
              " does not match the expected ", want);
  TORCH_CHECK(output.sizes().equals(input_.sizes()), op, ": output shape ", output.sizes(),
              " differs from the input shape ", input_.sizes());
  (void)to_rownorm_dtype(input_.scalar_type(), op);
  Tensor input = input_.dim() == 0 ? input_.view(1) : input_;
  Tensor out = output.dim() == 0 ? output.view(1) : output;
  const int64_t dim = at::maybe_wrap_dim(dim_, input.dim());
  if (input.numel() == 0) return;
  c10::DeviceGuard guard(input.device());
  if (dim == input.dim() - 1) {
    const Tensor in_c = input.contiguous();
    if (out.is_contiguous()) {
      forward_lastdim(in_c, out, is_log, op);
    } else {
      Tensor tmp = at::empty_like(out, out.options(), at::MemoryFormat::Contiguous);
      forward_lastdim(in_c, tmp, is_log, op);
      out.copy_(tmp);
    }
  } else {
    const Tensor in_t = input.movedim(dim, -1).contiguous();
    Tensor out_t = at::empty(in_t.sizes(), out.options());
    forward_lastdim(in_t, out_t, is_log, op);
    out.copy_(out_t.movedim(-1, dim));
  }
}

// host_softmax_backward, SoftMaxKernels.cpp:2180-2240: with half_to_float the
// gradient is Float and the input gradient Half.
void softmax_backward_entry(const Tensor& grad_, const Tensor& output_, int64_t dim_,
                            bool half_to_float, const Tensor& grad_input, bool is_log,
                            const char* op) {
  check_gpu(grad_, op, "grad_output");
  check_same_device(grad_, output_, op, "output");
  check_same_device(grad_, grad_input, op, "grad_input");
  TORCH_CHECK(grad_.scalar_type() == output_.scalar_type(), op, ": grad_output dtype ",
              grad_.scalar_type(), " differs from output dtype ", output_.scalar_type());
  if (half_to_float) {
    TORCH_CHECK(grad_.scalar_type() == at::kFloat && grad_input.scalar_type() == at::kHalf, op,
                ": expected input and grad types to match, or input to be at::Half and grad to "
                "be at::Float");
  } else {
    TORCH_CHECK(grad_input.scalar_type() == grad_.scalar_type(), op, ": grad_input dtype ",
                grad_input.scalar_type(), " differs from grad_output dtype ", grad_.scalar_type());
  }
  TORCH_CHECK(grad_.sizes().equals(output_.sizes()) && grad_input.sizes().equals(output_.sizes()),
              op, ": grad_output, output and grad_input must share a shape");
  (void)to_rownorm_dtype(grad_.scalar_type(), op);
  Tensor grad = grad_.dim() == 0 ? grad_.view(1) : grad_;
  Tensor y = output_.dim() == 0 ? output_.view(1) : output_;
  Tensor gi = grad_input.dim() == 0 ? grad_input.view(1) : grad_input;
  const int64_t dim = at::maybe_wrap_dim(dim_, grad.dim());
  if (grad.numel() == 0) return;
  c10::DeviceGuard guard(grad.device());
  if (dim == grad.dim() - 1) {
    const Tensor g_c = grad.contiguous();
    const Tensor y_c = y.contiguous();
    if (gi.is_contiguous()) {
      backward_lastdim(g_c, y_c, gi, is_log, op);
    } else {
      Tensor tmp = at::empty_like(gi, gi.options(), at::MemoryFormat::Contiguous);
      backward_lastdim(g_c, y_c, tmp, is_log, op);
      gi.copy_(tmp);
    }
  } else {
    const Tensor g_t = grad.movedim(dim, -1).contiguous();
    const Tensor y_t = y.movedim(dim, -1).contiguous();
    Tensor gi_t = at::empty(g_t.sizes(), gi.options());
    backward_lastdim(g_t, y_t, gi_t, is_log, op);
    gi.copy_(gi_t.movedim(-1, dim));
  }
}

Tensor alloc_forward_output(const Tensor& self, bool half_to_float) {
  return at::empty_like(self, self.options().dtype(half_to_float ? at::kFloat : self.scalar_type()),
                        at::MemoryFormat::Contiguous);
}

// SoftMax.cpp:44-55: half_to_float is implied by grad.dtype != input_dtype and
// only (Float grad, Half input) is legal.
bool backward_half_to_float(const Tensor& grad, at::ScalarType input_dtype) {
  const bool h2f = grad.scalar_type() != input_dtype;
  if (h2f) {
    TORCH_CHECK(grad.scalar_type() == at::kFloat && input_dtype == at::kHalf,
                "expected input and grad types to match, or input to be at::Half and grad to be "
                "at::Float");
  }
  return h2f;
}

}  // namespace

void _softmax_kernel(const Tensor& input, int64_t dim, bool half_to_float, const Tensor& output) {
  softmax_forward_entry(input, dim, half_to_float, output, false, "mi355x::_softmax");
}
void _log_softmax_kernel(const Tensor& input, int64_t dim, bool half_to_float,
                         const Tensor& output) {
  softmax_forward_entry(input, dim, half_to_float, output, true, "mi355x::_log_softmax");
}
void _softmax_backward_kernel(const Tensor& grad, const Tensor& output, int64_t dim,
                              bool half_to_float, const Tensor& grad_input) {
  softmax_backward_entry(grad, output, dim, half_to_float, grad_input, false,
                         "mi355x::_softmax_backward_data");
}
void _log_softmax_backward_kernel(const Tensor& grad, const Tensor& output, int64_t dim,
                                  bool half_to_float, const Tensor& grad_input) {
  softmax_backward_entry(grad, output, dim, half_to_float, grad_input, true,
                         "mi355x::_log_softmax_backward_data");
}

Tensor _softmax(const Tensor& self, int64_t dim, bool half_to_float) {
  check_gpu(self, "mi355x::_softmax", "self");
  Tensor out = alloc_forward_output(self, half_to_float);
  _softmax_kernel(self, dim, half_to_float, out);
  return out;
}
Tensor _log_softmax(const Tensor& self, int64_t dim, bool half_to_float) {
  check_gpu(self, "mi355x::_log_softmax", "self");
  Tensor out = alloc_forward_output(self, half_to_float);
  _log_softmax_kernel(self, dim, half_to_float, out);
  return out;
}
Tensor& _softmax_out(const Tensor& self, int64_t dim, bool half_to_float, Tensor& out) {
  at::native::resize_output(out, self.sizes());
  _softmax_kernel(self, dim, half_to_float, out);
  return out;
}
Tensor& _log_softmax_out(const Tensor& self, int64_t dim, bool half_to_float, Tensor& out) {
  at::native::resize_output(out, self.sizes());
  _log_softmax_kernel(self, dim, half_to_float, out);
  return out;
}

Tensor _softmax_backward_data(const Tensor& grad_output, const Tensor& output, int64_t dim,
                              at::ScalarType input_dtype) {
  const bool h2f = backward_half_to_float(grad_output, input_dtype);
  check_gpu(grad_output, "mi355x::_softmax_backward_data", "grad_output");
  Tensor gi = at::empty_like(grad_output, grad_output.options().dtype(input_dtype),
                             at::MemoryFormat::Contiguous);
  _softmax_backward_kernel(grad_output, output, dim, h2f, gi);
  return gi;
}
Tensor _log_softmax_backward_data(const Tensor& grad_output, const Tensor& output, int64_t dim,
                                  at::ScalarType input_dtype) {
  const bool h2f = backward_half_to_float(grad_output, input_dtype);
  check_gpu(grad_output, "mi355x::_log_softmax_backward_data", "grad_output");
  Tensor gi = at::empty_like(grad_output, grad_output.options().dtype(input_dtype),
                             at::MemoryFormat::Contiguous);
  _log_softmax_backward_kernel(grad_output, output, dim, h2f, gi);
  return gi;
}
Tensor& _softmax_backward_data_out(const Tensor& grad_output, const Tensor& output, int64_t dim,
                                   at::ScalarType input_dtype, Tensor& grad_input) {
  const bool h2f = backward_half_to_float(grad_output, input_dtype);
  at::native::resize_output(grad_input, grad_output.sizes());
  _softmax_backward_kernel(grad_output, output, dim, h2f, grad_input);
  return grad_input;
}
Tensor& _log_softmax_backward_data_out(const Tensor& grad_output, const Tensor& output,
                                       int64_t dim, at::ScalarType input_dtype,
                                       Tensor& grad_input) {
  const bool h2f = backward_half_to_float(grad_output, input_dtype);
  at::native::resize_output(grad_input, grad_output.sizes());
  _log_softmax_backward_kernel(grad_output, output, dim, h2f, grad_input);
  return grad_input;
}

}  // namespace mi355x
