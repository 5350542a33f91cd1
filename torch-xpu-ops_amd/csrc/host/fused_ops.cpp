// Fused residual add -> norm host operators: checks, output allocation, one call into the C ABI
// (mi355x_add_layer_norm_fwd & co. in include/mi355x_rownorm.h).  Shapes, saved statistics and
// output masks follow the unfused operators in norm_ops.cpp, i.e. the contracts of the
// reference's src/ATen/native/xpu/LayerNorm.cpp:35-305.
#include <ATen/core/grad_mode.h>
#include "fused_ops.h"

#include <ATen/native/layer_norm.h>
#include <limits>

#include "host_common.h"

namespace mi355x {
namespace {

using at::Tensor;

Tensor defined_or_empty(const std::optional<Tensor>& t) {
  return (t.has_value() && t->defined()) ? *t : Tensor();
}

std::vector<int64_t> stat_shape_of(const Tensor& input, size_t normalized_ndim) {
  const size_t axis = input.dim() - normalized_ndim;
  std::vector<int64_t> shape(input.sizes().begin(), input.sizes().begin() + axis);
  shape.resize(input.dim(), 1);
  return shape;
}

rownorm_dtype weight_dtype(const Tensor& X, const Tensor& gamma, const Tensor& beta,
                           const char* op) {
  const Tensor& w = gamma.defined() ? gamma : beta;
  if (!w.defined()) return to_rownorm_dtype(X.scalar_type(), op);
  if (gamma.defined() && beta.defined()) {
    TORCH_CHECK(gamma.scalar_type() == beta.scalar_type(), op,
                ": weight and bias must share a dtype, got ", gamma.scalar_type(), " and ",
                beta.scalar_type());
  }
  TORCH_CHECK(w.scalar_type() == X.scalar_type() || w.scalar_type() == at::kFloat, op,
              ": weight dtype must equal the input dtype or be float32, got ", w.scalar_type(),
              " with input ", X.scalar_type());
  return to_rownorm_dtype(w.scalar_type(), op);
}

// The dtype y is written in: the input dtype, or a 16-bit type for a float32 input.
at::ScalarType check_out_dtype(const Tensor& input, std::optional<at::ScalarType> out_dtype,
                               const char* op) {
  const at::ScalarType want = out_dtype.value_or(input.scalar_type());
  TORCH_CHECK(want == input.scalar_type() ||
                  (input.scalar_type() == at::kFloat &&
                   (want == at::kHalf || want == at::kBFloat16)),
              op, ": out_dtype must be the input dtype, or Half / BFloat16 for a Float input; got ",
              want, " for input ", input.scalar_type());
  return want;
}

struct Forward {
  Tensor X, R, H, Y;
};

// Common part of the two forwards: checks, contiguous operands, h and y.
// These operators are registered for every dispatch key with no autograd formula
// of their own: called on a tensor that requires a gradient they would hand back
// outputs cut off from the graph without a word.  The differentiable forms are
// torch_xpu_ops_amd.fused.add_rms_norm / add_layer_norm (autograd.Function, whose
// forward runs with gradient recording off and so passes this check).
void check_no_grad_wanted(const Tensor& t, const char* op, const char* name) {
  TORCH_CHECK(!(t.defined() && at::GradMode::is_enabled() && t.requires_grad()), op, ": `", name,
              "` requires a gradient, but this operator records no autograd graph; call "
              "fused.add_rms_norm / fused.add_layer_norm (differentiable), or detach the "
              "tensor / use torch.no_grad()");
}

Forward prepare_forward(const Tensor& input, const Tensor& residual,
                        std::optional<at::ScalarType> out_dtype, bool inplace, const char* op) {
  check_no_grad_wanted(input, op, "input");
  check_no_grad_wanted(residual, op, "residual");
  check_gpu(input, op, "input");
  check_same_device(input, residual, op, "residual");
  TORCH_CHECK(residual.defined() && residual.sizes().equals(input.sizes()) &&
                  residual.scalar_type() == input.scalar_type(),
              op, ": residual must have the shape and dtype of input, got ", residual.sizes(), " ",
              residual.scalar_type(), " for ", input.sizes(), " ", input.scalar_type());
  (void)to_rownorm_dtype(input.scalar_type(), op);
  Forward f;
  f.X = input.contiguous();
  if (inplace) {
    TORCH_CHECK(residual.is_contiguous(), op,
                ": the in-place form needs a contiguous residual tensor");
    f.R = residual;
    f.H = residual;
  } else {
    f.R = residual.contiguous();
    f.H = at::empty_like(f.X, f.X.options(), at::MemoryFormat::Contiguous);
  }
  f.Y = at::empty_like(f.X, f.X.options().dtype(check_out_dtype(input, out_dtype, op)),
                       at::MemoryFormat::Contiguous);
  return f;
}

std::tuple<Tensor, Tensor, Tensor, Tensor> add_layer_norm_impl(
    const Tensor& input, const Tensor& residual, at::IntArrayRef normalized_shape,
    const std::optional<Tensor>& weight_opt, const std::optional<Tensor>& bias_opt, double eps,
    std::optional<at::ScalarType> out_dtype, bool inplace) {
  static const char* op = "mi355x::add_layer_norm";
  const Tensor weight = defined_or_empty(weight_opt);
  const Tensor bias = defined_or_empty(bias_opt);
  check_no_grad_wanted(weight, op, "weight");
  check_no_grad_wanted(bias, op, "bias");
  check_same_device(input, weight, op, "weight");
  check_same_device(input, bias, op, "bias");
  const auto [M, N] = at::native::_check_layer_norm_inputs(input, normalized_shape, weight, bias);
  c10::DeviceGuard guard(input.device());
  Forward f = prepare_forward(input, residual, out_dtype, inplace, op);
  const Tensor gamma = weight.defined() ? weight.contiguous() : weight;
  const Tensor beta = bias.defined() ? bias.contiguous() : bias;
  Tensor mean = at::empty({M}, f.X.options().dtype(at::kFloat));
  Tensor rstd = at::empty({M}, f.X.options().dtype(at::kFloat));
  if (M > 0 && N > 0) {
    check_status(
        mi355x_add_layer_norm_fwd(f.X.const_data_ptr(), f.R.const_data_ptr(), ptr_or_null(gamma),
                                  ptr_or_null(beta), f.H.mutable_data_ptr(),
                                  f.Y.mutable_data_ptr(), (float*)mean.mutable_data_ptr(),
                                  (float*)rstd.mutable_data_ptr(), M, N, (float)eps,
                                  to_rownorm_dtype(f.X.scalar_type(), op),
                                  weight_dtype(f.X, gamma, beta, op),
                                  to_rownorm_dtype(f.Y.scalar_type(), op), current_stream(f.X)),
        op);
  } else if (M > 0) {
    mean.zero_();
    rstd.fill_(std::numeric_limits<float>::quiet_NaN());
  }
  const auto stat_shape = stat_shape_of(input, normalized_shape.size());
  return std::make_tuple(std::move(f.Y), std::move(f.H), mean.view(stat_shape),
                         rstd.view(stat_shape));
}

std::tuple<Tensor, Tensor, Tensor> add_rms_norm_impl(const Tensor& input, const Tensor& residual,
                                                     at::IntArrayRef normalized_shape,
                                                     const std::optional<Tensor>& weight_opt,
                                                     std::optional<double> eps_opt,
                                                     std::optional<at::ScalarType> out_dtype,
                                                     bool inplace) {
  static const char* op = "mi355x::add_rms_norm";
  const Tensor weight = defined_or_empty(weight_opt);
  check_no_grad_wanted(weight, op, "weight");
  check_same_device(input, weight, op, "weight");
  const auto [M, N] =
      at::native::_check_layer_norm_inputs(input, normalized_shape, weight, weight);
  c10::DeviceGuard guard(input.device());
  Forward f = prepare_forward(input, residual, out_dtype, inplace, op);
  const Tensor gamma = weight.defined() ? weight.contiguous() : weight;
  const double eps = eps_opt.value_or((double)std::numeric_limits<float>::epsilon());
  Tensor rstd = at::empty({M}, f.X.options().dtype(at::kFloat));
  if (M > 0 && N > 0) {
    check_status(
        mi355x_add_rms_norm_fwd(f.X.const_data_ptr(), f.R.const_data_ptr(), ptr_or_null(gamma),
                                f.H.mutable_data_ptr(), f.Y.mutable_data_ptr(),
                                (float*)rstd.mutable_data_ptr(), M, N, (float)eps,
                                to_rownorm_dtype(f.X.scalar_type(), op),
                                weight_dtype(f.X, gamma, Tensor(), op),
                                to_rownorm_dtype(f.Y.scalar_type(), op), current_stream(f.X)),
        op);
  } else if (M > 0) {
    rstd.fill_(std::numeric_limits<float>::quiet_NaN());
  }
  return std::make_tuple(std::move(f.Y), std::move(f.H),
                         rstd.view(stat_shape_of(input, normalized_shape.size())));
}

}  // namespace

std::tuple<Tensor, Tensor, Tensor, Tensor> add_layer_norm(
    const Tensor& input, const Tensor& residual, at::IntArrayRef normalized_shape,
    const std::optional<Tensor>& weight_opt, const std::optional<Tensor>& bias_opt, double eps,
    std::optional<at::ScalarType> out_dtype) {
  return add_layer_norm_impl(input, residual, normalized_shape, weight_opt, bias_opt, eps,
                             out_dtype, false);
}

std::tuple<Tensor, Tensor, Tensor> add_layer_norm_(
    const Tensor& input, Tensor& residual, at::IntArrayRef normalized_shape,
    const std::optional<Tensor>& weight_opt, const std::optional<Tensor>& bias_opt, double eps,
    std::optional<at::ScalarType> out_dtype) {
  auto [y, h, mean, rstd] = add_layer_norm_impl(input, residual, normalized_shape, weight_opt,
                                                bias_opt, eps, out_dtype, true);
  return std::make_tuple(std::move(y), std::move(mean), std::move(rstd));
}

std::tuple<Tensor, Tensor, Tensor> add_rms_norm(const Tensor& input, const Tensor& residual,
                                                at::IntArrayRef normalized_shape,
                                                const std::optional<Tensor>& weight_opt,
                                                std::optional<double> eps_opt,
                                                std::optional<at::ScalarType> out_dtype) {
  return add_rms_norm_impl(input, residual, normalized_shape, weight_opt, eps_opt, out_dtype,
                           false);
}

std::tuple<Tensor, Tensor> add_rms_norm_(const Tensor& input, Tensor& residual,
                                         at::IntArrayRef normalized_shape,
                                         const std::optional<Tensor>& weight_opt,
                                         std::optional<double> eps_opt,
                                         std::optional<at::ScalarType> out_dtype) {
  auto [y, h, rstd] = add_rms_norm_impl(input, residual, normalized_shape, weight_opt, eps_opt,
                                        out_dtype, true);
  return std::make_tuple(std::move(y), std::move(rstd));
}

namespace {

// Checks shared by the two backwards; returns the contiguous (grad_y, grad_h, h).
std::tuple<Tensor, Tensor, Tensor> prepare_backward(const Tensor& grad_y,
                                                    const std::optional<Tensor>& grad_h_opt,
                                                    const Tensor& h, const char* op) {
  check_gpu(h, op, "h");
  check_same_device(h, grad_y, op, "grad_y");
  (void)to_rownorm_dtype(h.scalar_type(), op);
  TORCH_CHECK(grad_y.scalar_type() == h.scalar_type() && grad_y.sizes().equals(h.sizes()), op,
              ": grad_y must have the shape and dtype of h (the backward has no output cast), got ",
              grad_y.sizes(), " ", grad_y.scalar_type(), " for ", h.sizes(), " ", h.scalar_type());
  Tensor gh = defined_or_empty(grad_h_opt);
  if (gh.defined()) {
    check_same_device(h, gh, op, "grad_h");
    TORCH_CHECK(gh.scalar_type() == h.scalar_type() && gh.sizes().equals(h.sizes()), op,
                ": grad_h must have the shape and dtype of h");
    gh = gh.contiguous();
  }
  return std::make_tuple(grad_y.contiguous(), gh, h.contiguous());
}

}  // namespace

std::tuple<Tensor, Tensor, Tensor> add_layer_norm_backward(
    const Tensor& grad_y, const std::optional<Tensor>& grad_h_opt, const Tensor& h,
    at::IntArrayRef normalized_shape, const Tensor& mean, const Tensor& rstd,
    const std::optional<Tensor>& weight_opt, const std::optional<Tensor>& bias_opt,
    std::array<bool, 3> output_mask) {
  static const char* op = "mi355x::add_layer_norm_backward";
  const Tensor weight = defined_or_empty(weight_opt);
  const Tensor bias = defined_or_empty(bias_opt);
  const auto [M, N] = at::native::_check_layer_norm_inputs(h, normalized_shape, weight, bias);
  c10::DeviceGuard guard(h.device());
  auto [dY, dHin, H] = prepare_backward(grad_y, grad_h_opt, h, op);
  check_same_device(h, mean, op, "mean");
  check_same_device(h, rstd, op, "rstd");
  TORCH_CHECK(mean.scalar_type() == at::kFloat && rstd.scalar_type() == at::kFloat &&
                  mean.numel() == M && rstd.numel() == M,
              op, ": mean and rstd must be the float32 statistics the forward returned");
  const Tensor gamma = weight.defined() ? weight.contiguous() : weight;
  const Tensor mc = mean.contiguous(), rc = rstd.contiguous();
  const rownorm_dtype xd = to_rownorm_dtype(H.scalar_type(), op);
  const rownorm_dtype wd = weight_dtype(H, gamma, bias, op);
  Tensor dH, dgamma, dbeta;
  if (output_mask[0]) dH = at::empty_like(H, H.options(), at::MemoryFormat::Contiguous);
  if (output_mask[1] && gamma.defined())
    dgamma = M > 0 ? at::empty_like(gamma, at::MemoryFormat::Contiguous)
                   : at::zeros_like(gamma, at::MemoryFormat::Contiguous);
  if (output_mask[2] && bias.defined())
    dbeta = M > 0 ? at::empty_like(bias, at::MemoryFormat::Contiguous)
                  : at::zeros_like(bias, at::MemoryFormat::Contiguous);
  if (M > 0 && N > 0) {
    const size_t ws_bytes = mi355x_layer_norm_bwd_workspace_bytes(M, N, xd, wd, dgamma.defined(),
                                                                  dbeta.defined());
    Tensor ws;
    if (ws_bytes > 0) ws = at::empty({(int64_t)ws_bytes}, H.options().dtype(at::kByte));
    check_status(mi355x_add_layer_norm_bwd(
                     dY.const_data_ptr(), ptr_or_null(dHin), H.const_data_ptr(),
                     (const float*)mc.const_data_ptr(), (const float*)rc.const_data_ptr(),
                     ptr_or_null(gamma), mut_ptr_or_null(&dH), mut_ptr_or_null(&dgamma),
                     mut_ptr_or_null(&dbeta), ws.defined() ? ws.mutable_data_ptr() : nullptr,
                     ws_bytes, M, N, xd, wd, current_stream(H)),
                 op);
  } else if (dH.defined() && dHin.defined()) {
    dH.copy_(dHin);
  }
  return std::make_tuple(std::move(dH), std::move(dgamma), std::move(dbeta));
}

std::tuple<Tensor, Tensor> add_rms_norm_backward(const Tensor& grad_y,
                                                 const std::optional<Tensor>& grad_h_opt,
                                                 const Tensor& h,
                                                 at::IntArrayRef normalized_shape,
                                                 const Tensor& rstd,
                                                 const std::optional<Tensor>& weight_opt,
                                                 std::array<bool, 2> output_mask) {
  static const char* op = "mi355x::add_rms_norm_backward";
  const Tensor weight = defined_or_empty(weight_opt);
  const auto [M, N] = at::native::_check_layer_norm_inputs(h, normalized_shape, weight, weight);
  c10::DeviceGuard guard(h.device());
  auto [dY, dHin, H] = prepare_backward(grad_y, grad_h_opt, h, op);
  check_same_device(h, rstd, op, "rstd");
  TORCH_CHECK(rstd.scalar_type() == at::kFloat && rstd.numel() == M, op,
              ": rstd must be the float32 statistic the forward returned");
  const Tensor gamma = weight.defined() ? weight.contiguous() : weight;
  const Tensor rc = rstd.contiguous();
  const rownorm_dtype xd = to_rownorm_dtype(H.scalar_type(), op);
  const rownorm_dtype wd = weight_dtype(H, gamma, Tensor(), op);
  Tensor dH, dgamma;
  if (output_mask[0]) dH = at::empty_like(H, H.options(), at::MemoryFormat::Contiguous);
  if (output_mask[1] && gamma.defined())
    dgamma = M > 0 ? at::empty_like(gamma, at::MemoryFormat::Contiguous)
                   : at::zeros_like(gamma, at::MemoryFormat::Contiguous);
  if (M > 0 && N > 0) {
    const size_t ws_bytes = mi355x_rms_norm_bwd_workspace_bytes(M, N, xd, wd, dgamma.defined());
    Tensor ws;
    if (ws_bytes > 0) ws = at::empty({(int64_t)ws_bytes}, H.options().dtype(at::kByte));
    check_status(mi355x_add_rms_norm_bwd(dY.const_data_ptr(), ptr_or_null(dHin),
                                         H.const_data_ptr(), (const float*)rc.const_data_ptr(),
                                         ptr_or_null(gamma), mut_ptr_or_null(&dH),
                                         mut_ptr_or_null(&dgamma),
                                         ws.defined() ? ws.mutable_data_ptr() : nullptr, ws_bytes,
                                         M, N, xd, wd, current_stream(H)),
                 op);
  } else if (dH.defined() && dHin.defined()) {
    dH.copy_(dHin);
  }
  return std::make_tuple(std::move(dH), std::move(dgamma));
}

}  // namespace mi355x
