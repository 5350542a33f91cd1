// softmax / log_softmax host operators.  Contracts follow the reference's
// src/ATen/native/xpu/SoftMax.cpp:22-100 and the host_softmax /
// host_softmax_backward entry code in SoftMaxKernels.cpp:2125-2276.
//
// The kernels work on dense tensors: the innermost-dimension kernels for
// dim == -1, the [outer, dim, inner] kernels for any other dimension (no
// transposing copies).  Only a masked softmax over a non-innermost dimension
// moves that dimension last first.
#include "softmax_ops.h"

#include <ATen/WrapDimUtils.h>
#include <ATen/native/Resize.h>
#include <ATen/ops/_log_softmax_backward_data_cuda_dispatch.h>
#include <ATen/ops/_log_softmax_cuda_dispatch.h>
#include <ATen/ops/_masked_softmax_backward_cuda_dispatch.h>
#include <ATen/ops/_masked_softmax_cuda_dispatch.h>
#include <ATen/ops/_safe_softmax_native.h>
#include <ATen/ops/_softmax_backward_data_cuda_dispatch.h>
#include <ATen/ops/_softmax_cuda_dispatch.h>

#include "host_common.h"

namespace mi355x {
namespace {

using at::Tensor;

enum class Mode { kSoftmax, kLogSoftmax, kSafeSoftmax };

// Forward over dimension `dim` of the dense tensor `in` into the dense `out`.
void forward_dense(const Tensor& in, const Tensor& out, int64_t dim, Mode mode, const char* op) {
  int64_t outer = 1, inner = 1;
  for (int64_t i = 0; i < dim; ++i) outer *= in.size(i);
  for (int64_t i = dim + 1; i < in.dim(); ++i) inner *= in.size(i);
  const int abi_mode = mode == Mode::kSafeSoftmax  ? ROWNORM_SAFE_SOFTMAX
                       : mode == Mode::kLogSoftmax ? ROWNORM_LOG_SOFTMAX
                                                   : ROWNORM_SOFTMAX;
  check_status(mi355x_softmax_strided_fwd(in.const_data_ptr(), out.mutable_data_ptr(), outer,
                                          in.size(dim), inner,
                                          to_rownorm_dtype(in.scalar_type(), op),
                                          to_rownorm_dtype(out.scalar_type(), op), abi_mode,
                                          current_stream(in)),
               op);
}

void backward_dense(const Tensor& grad, const Tensor& y, const Tensor& gi, int64_t dim,
                    bool is_log, const char* op) {
  int64_t outer = 1, inner = 1;
  for (int64_t i = 0; i < dim; ++i) outer *= y.size(i);
  for (int64_t i = dim + 1; i < y.dim(); ++i) inner *= y.size(i);
  check_status(mi355x_softmax_strided_bwd(grad.const_data_ptr(), y.const_data_ptr(),
                                          gi.mutable_data_ptr(), outer, y.size(dim), inner,
                                          to_rownorm_dtype(grad.scalar_type(), op),
                                          to_rownorm_dtype(gi.scalar_type(), op),
                                          is_log ? ROWNORM_LOG_SOFTMAX : ROWNORM_SOFTMAX,
                                          current_stream(y)),
               op);
}

// host_softmax, SoftMaxKernels.cpp:2125-2178: half_to_float needs a Half
// input (:2131-2135); 0-dim tensors are viewed as [1] (:2143-2144); an empty
// tensor is a no-op (:2150).
void softmax_forward_entry(const Tensor& input_, int64_t dim_, bool half_to_float,
                           const Tensor& output, Mode mode, const char* op) {
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
  const Tensor in_c = input.contiguous();
  if (out.is_contiguous()) {
    forward_dense(in_c, out, dim, mode, op);
  } else {
    Tensor tmp = at::empty_like(out, out.options(), at::MemoryFormat::Contiguous);
    forward_dense(in_c, tmp, dim, mode, op);
    out.copy_(tmp);
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
  const Tensor g_c = grad.contiguous();
  const Tensor y_c = y.contiguous();
  if (gi.is_contiguous()) {
    backward_dense(g_c, y_c, gi, dim, is_log, op);
  } else {
    Tensor tmp = at::empty_like(gi, gi.options(), at::MemoryFormat::Contiguous);
    backward_dense(g_c, y_c, tmp, dim, is_log, op);
    gi.copy_(tmp);
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

// How a boolean mask lines up with the rows of a dense tensor whose softmax
// dimension is innermost: data row r reads mask row (r / div) * stride + r % mod.
struct MaskLayout {
  Tensor mask;  // dense [mask_rows, N] bool
  int64_t mask_rows, div, stride, mod;
};

// The shapes masked_softmax_kernel accepts (SoftMaxKernels.cpp:2315-2338): the
// input's own shape, a [B, T] key-padding mask (mask_type 1) or a [T, T] mask
// (mask_type 0) under a [B, H, T, T] input.  The two small masks are read in
// place; any other broadcastable mask is expanded once.
MaskLayout mask_layout_lastdim(const Tensor& input, const Tensor& mask, bool is_BxT,
                               bool is_TxT) {
  const int64_t N = input.size(-1);
  const int64_t rows = N == 0 ? 0 : input.numel() / N;
  if (is_BxT) {
    return {mask.contiguous(), mask.size(0), input.size(1) * input.size(2), 1, 1};
  }
  if (is_TxT) {
    return {mask.contiguous(), mask.size(0), 1, 0, mask.size(0)};
  }
  return {mask.expand(input.sizes()).contiguous(), rows, 1, 1, 1};
}

}  // namespace

// _safe_softmax_kernel, SoftMaxKernels.cpp:2278-2299.
Tensor _safe_softmax_kernel(const Tensor& self, int64_t dim, bool half_to_float) {
  check_gpu(self, "mi355x::_safe_softmax", "self");
  Tensor out = alloc_forward_output(self, half_to_float);
  softmax_forward_entry(self, dim, half_to_float, out, Mode::kSafeSoftmax,
                        "mi355x::_safe_softmax");
  return out;
}

// _safe_softmax_xpu, SoftMax.cpp:102-110: Half -> Float is fused into the
// kernel, any other dtype request converts the input first.
Tensor _safe_softmax(const Tensor& self, int64_t dim, std::optional<at::ScalarType> dtype) {
  check_gpu(self, "mi355x::_safe_softmax", "self");
  if (delegated_dtype(self) || (self.is_cuda() && dtype == at::kDouble)) {
    // ATen's composite formula; the softmax inside it comes back here and is delegated
    warn_delegated("mi355x::_safe_softmax");
    return at::native::_safe_softmax(self, dim, dtype);
  }
  if (self.scalar_type() == at::kHalf && dtype == at::kFloat)
    return _safe_softmax_kernel(self, dim, true);
  const Tensor converted = dtype.has_value() ? self.toType(dtype.value()) : self;
  return _safe_softmax_kernel(converted, dim, false);
}

// masked_softmax_kernel, SoftMaxKernels.cpp:2301-2359.
Tensor masked_softmax_kernel(const Tensor& input_, const Tensor& mask_,
                             std::optional<int64_t> dim_, std::optional<int64_t> mask_type_) {
  const char* op = "mi355x::_masked_softmax";
  TORCH_CHECK(mask_.scalar_type() == at::kBool, "Mask should be a boolean tensor");
  TORCH_CHECK(mask_type_.has_value(), "Mask Type should be defined");
  const int64_t mask_type = mask_type_.value();
  TORCH_CHECK(mask_type == 0 || mask_type == 1 || mask_type == 2,
              "Mask Type should be 0 (src_mask), 1 (src_key_padding_mask), or 2 (default_mask)");
  const bool is_BxT = mask_type == 1 && input_.dim() == 4 && mask_.dim() == 2 &&
                      input_.size(0) == mask_.size(0) && input_.size(2) == mask_.size(1) &&
                      input_.size(3) == mask_.size(1);
  const bool is_TxT = mask_type == 0 && input_.dim() == 4 && mask_.dim() == 2 &&
                      input_.size(3) == mask_.size(1) && input_.size(2) == mask_.size(0) &&
                      mask_.size(0) == mask_.size(1);
  TORCH_CHECK(mask_.sizes() == input_.sizes() || is_BxT || is_TxT,
              "Mask shape should match input. mask: ", mask_.sizes(), " input: ", input_.sizes());
  check_gpu(input_, op, "input");
  check_same_device(input_, mask_, op, "mask");
  const rownorm_dtype dt = to_rownorm_dtype(input_.scalar_type(), op);
  Tensor output = at::empty_like(input_, input_.options(), at::MemoryFormat::Contiguous);
  Tensor input = input_.dim() == 0 ? input_.view(1) : input_;
  Tensor mask = mask_.dim() == 0 ? mask_.view(1) : mask_;
  Tensor out = output.dim() == 0 ? output.view(1) : output;
  const int64_t dim =
      dim_.has_value() ? at::maybe_wrap_dim(dim_.value(), input.dim()) : input.dim() - 1;
  if (input.numel() == 0) return output;
  c10::DeviceGuard guard(input.device());
  auto run = [&](const Tensor& in, const MaskLayout& ml, const Tensor& o) {
    const int64_t N = in.size(-1);
    check_status(mi355x_masked_softmax_fwd(in.const_data_ptr(), ml.mask.const_data_ptr(),
                                           o.mutable_data_ptr(), in.numel() / N, N, ml.mask_rows,
                                           ml.div, ml.stride, ml.mod, dt, current_stream(in)),
                 op);
  };
  if (dim == input.dim() - 1) {
    const Tensor in_c = input.contiguous();
    run(in_c, mask_layout_lastdim(in_c, mask, is_BxT, is_TxT), out);
  } else {
    // the mask follows the input through the transposition
    Tensor full = is_BxT ? mask.view({mask.size(0), 1, 1, mask.size(1)}) : mask;
    full = full.expand(input.sizes());
    const Tensor in_t = input.movedim(dim, -1).contiguous();
    const Tensor mask_t = full.movedim(dim, -1).contiguous();
    Tensor out_t = at::empty(in_t.sizes(), out.options());
    run(in_t, MaskLayout{mask_t, in_t.numel() / in_t.size(-1), 1, 1, 1}, out_t);
    out.copy_(out_t.movedim(-1, dim));
  }
  return output;
}

// masked_softmax_backward_kernel, SoftMaxKernels.cpp:2361-2401.
Tensor masked_softmax_backward_kernel(const Tensor& grad_, const Tensor& output_,
                                      const Tensor& mask_, std::optional<int64_t> dim_) {
  const char* op = "mi355x::_masked_softmax_backward";
  check_gpu(grad_, op, "grad_output");
  check_same_device(grad_, output_, op, "output");
  check_same_device(grad_, mask_, op, "mask");
  Tensor grad_input = at::empty_like(grad_, grad_.options(), at::MemoryFormat::Contiguous);
  if (grad_.numel() == 0) return grad_input;
  Tensor grad = grad_.contiguous();
  Tensor output = output_.contiguous();
  Tensor mask = mask_.contiguous();
  const int64_t dim =
      dim_.has_value() ? at::maybe_wrap_dim(dim_.value(), output.dim()) : output.dim() - 1;
  grad = grad.dim() == 0 ? grad.view(1) : grad;
  mask = mask.dim() == 0 ? mask.view(1) : mask;
  output = output.dim() == 0 ? output.view(1) : output;
  Tensor gi = grad_input.dim() == 0 ? grad_input.view(1) : grad_input;
  TORCH_CHECK(dim >= 0 && dim < grad.dim(),
              "dim must be non-negative and less than input dimensions");
  TORCH_CHECK(grad.sizes() == mask.sizes(), "Mask shape should match grad shape");
  TORCH_CHECK(grad.sizes() == output.sizes(), op, ": grad_output and output must share a shape");
  TORCH_CHECK(mask.scalar_type() == at::kBool, "Mask should be a boolean tensor");
  TORCH_CHECK(grad.scalar_type() == output.scalar_type(), op, ": grad_output dtype ",
              grad.scalar_type(), " differs from output dtype ", output.scalar_type());
  const rownorm_dtype dt = to_rownorm_dtype(grad.scalar_type(), op);
  c10::DeviceGuard guard(grad.device());
  auto run = [&](const Tensor& g, const Tensor& y, const Tensor& m, const Tensor& o) {
    const int64_t N = g.size(-1);
    const int64_t rows = g.numel() / N;
    check_status(mi355x_masked_softmax_bwd(g.const_data_ptr(), y.const_data_ptr(),
                                           m.const_data_ptr(), o.mutable_data_ptr(), rows, N, rows,
                                           1, 1, 1, dt, current_stream(g)),
                 op);
  };
  if (dim == grad.dim() - 1) {
    run(grad, output, mask, gi);
  } else {
    const Tensor g_t = grad.movedim(dim, -1).contiguous();
    const Tensor y_t = output.movedim(dim, -1).contiguous();
    const Tensor m_t = mask.movedim(dim, -1).contiguous();
    Tensor gi_t = at::empty(g_t.sizes(), gi.options());
    run(g_t, y_t, m_t, gi_t);
    gi.copy_(gi_t.movedim(-1, dim));
  }
  return grad_input;
}

// masked_softmax_xpu / masked_softmax_backward_xpu, SoftMax.cpp:112-126.
Tensor _masked_softmax(const Tensor& self, const Tensor& mask, std::optional<int64_t> dim,
                       std::optional<int64_t> mask_type) {
  if (delegated_dtype(self)) {
    warn_delegated("mi355x::_masked_softmax");
    return at::cuda::_masked_softmax(self, mask, dim, mask_type);
  }
  return masked_softmax_kernel(self, mask, dim, mask_type);
}
Tensor _masked_softmax_backward(const Tensor& grad_output, const Tensor& output,
                                const Tensor& mask, std::optional<int64_t> dim) {
  if (delegated_dtype(grad_output)) {
    warn_delegated("mi355x::_masked_softmax_backward");
    return at::cuda::_masked_softmax_backward(grad_output, output, mask, dim);
  }
  return masked_softmax_backward_kernel(grad_output, output, mask, dim);
}

void _softmax_kernel(const Tensor& input, int64_t dim, bool half_to_float, const Tensor& output) {
  softmax_forward_entry(input, dim, half_to_float, output, Mode::kSoftmax, "mi355x::_softmax");
}
void _log_softmax_kernel(const Tensor& input, int64_t dim, bool half_to_float,
                         const Tensor& output) {
  softmax_forward_entry(input, dim, half_to_float, output, Mode::kLogSoftmax,
                        "mi355x::_log_softmax");
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
  if (delegated_dtype(self)) {
    warn_delegated("mi355x::_softmax");
    return at::cuda::_softmax(self, dim, half_to_float);
  }
  check_gpu(self, "mi355x::_softmax", "self");
  Tensor out = alloc_forward_output(self, half_to_float);
  _softmax_kernel(self, dim, half_to_float, out);
  return out;
}
Tensor _log_softmax(const Tensor& self, int64_t dim, bool half_to_float) {
  if (delegated_dtype(self)) {
    warn_delegated("mi355x::_log_softmax");
    return at::cuda::_log_softmax(self, dim, half_to_float);
  }
  check_gpu(self, "mi355x::_log_softmax", "self");
  Tensor out = alloc_forward_output(self, half_to_float);
  _log_softmax_kernel(self, dim, half_to_float, out);
  return out;
}
Tensor& _softmax_out(const Tensor& self, int64_t dim, bool half_to_float, Tensor& out) {
  if (delegated_dtype(self)) {
    warn_delegated("mi355x::_softmax.out");
    return at::cuda::_softmax_out(out, self, dim, half_to_float);
  }
  at::native::resize_output(out, self.sizes());
  _softmax_kernel(self, dim, half_to_float, out);
  return out;
}
Tensor& _log_softmax_out(const Tensor& self, int64_t dim, bool half_to_float, Tensor& out) {
  if (delegated_dtype(self)) {
    warn_delegated("mi355x::_log_softmax.out");
    return at::cuda::_log_softmax_out(out, self, dim, half_to_float);
  }
  at::native::resize_output(out, self.sizes());
  _log_softmax_kernel(self, dim, half_to_float, out);
  return out;
}

Tensor _softmax_backward_data(const Tensor& grad_output, const Tensor& output, int64_t dim,
                              at::ScalarType input_dtype) {
  if (delegated_dtype(grad_output)) {
    warn_delegated("mi355x::_softmax_backward_data");
    return at::cuda::_softmax_backward_data(grad_output, output, dim, input_dtype);
  }
  const bool h2f = backward_half_to_float(grad_output, input_dtype);
  check_gpu(grad_output, "mi355x::_softmax_backward_data", "grad_output");
  Tensor gi = at::empty_like(grad_output, grad_output.options().dtype(input_dtype),
                             at::MemoryFormat::Contiguous);
  _softmax_backward_kernel(grad_output, output, dim, h2f, gi);
  return gi;
}
Tensor _log_softmax_backward_data(const Tensor& grad_output, const Tensor& output, int64_t dim,
                                  at::ScalarType input_dtype) {
  if (delegated_dtype(grad_output)) {
    warn_delegated("mi355x::_log_softmax_backward_data");
    return at::cuda::_log_softmax_backward_data(grad_output, output, dim, input_dtype);
  }
  const bool h2f = backward_half_to_float(grad_output, input_dtype);
  check_gpu(grad_output, "mi355x::_log_softmax_backward_data", "grad_output");
  Tensor gi = at::empty_like(grad_output, grad_output.options().dtype(input_dtype),
                             at::MemoryFormat::Contiguous);
  _log_softmax_backward_kernel(grad_output, output, dim, h2f, gi);
  return gi;
}
Tensor& _softmax_backward_data_out(const Tensor& grad_output, const Tensor& output, int64_t dim,
                                   at::ScalarType input_dtype, Tensor& grad_input) {
  if (delegated_dtype(grad_output)) {
    warn_delegated("mi355x::_softmax_backward_data.out");
    return at::cuda::_softmax_backward_data_out(grad_input, grad_output, output, dim, input_dtype);
  }
  const bool h2f = backward_half_to_float(grad_output, input_dtype);
  at::native::resize_output(grad_input, grad_output.sizes());
  _softmax_backward_kernel(grad_output, output, dim, h2f, grad_input);
  return grad_input;
}
Tensor& _log_softmax_backward_data_out(const Tensor& grad_output, const Tensor& output,
                                       int64_t dim, at::ScalarType input_dtype,
                                       Tensor& grad_input) {
  if (delegated_dtype(grad_output)) {
    warn_delegated("mi355x::_log_softmax_backward_data.out");
    return at::cuda::_log_softmax_backward_data_out(grad_input, grad_output, output, dim,
                                                    input_dtype);
  }
  const bool h2f = backward_half_to_float(grad_output, input_dtype);
  at::native::resize_output(grad_input, grad_output.sizes());
  _log_softmax_backward_kernel(grad_output, output, dim, h2f, grad_input);
  return grad_input;
}

}  // namespace mi355x
