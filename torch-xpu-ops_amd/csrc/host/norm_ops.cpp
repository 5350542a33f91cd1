// LayerNorm / RMSNorm host operators: shape checks, output allocation, saved
// statistics layout, then one call into the C ABI.  Contracts follow the
// reference's src/ATen/native/xpu/LayerNorm.cpp (cited per function).
#include "dispatch_stub_slot.h"
#include "norm_ops.h"

#include <ATen/native/layer_norm.h>
#include <ATen/ops/_fused_rms_norm_backward_cuda_dispatch.h>
#include <ATen/ops/_fused_rms_norm_cuda_dispatch.h>
#include <ATen/ops/native_layer_norm_backward_cuda_dispatch.h>
#include <ATen/ops/native_layer_norm_cuda_dispatch.h>
#include <limits>

#include "host_common.h"

namespace mi355x {
namespace {

using at::Tensor;

Tensor defined_or_empty(const std::optional<Tensor>& t) {
  return (t.has_value() && t->defined()) ? *t : Tensor();
}

// input.shape[:axis] + [1] * len(normalized_shape): the shape mean/rstd are
// returned in (LayerNorm.cpp:82-94, 239-250).
std::vector<int64_t> stat_shape_of(const Tensor& input, size_t normalized_ndim) {
  const size_t axis = input.dim() - normalized_ndim;
  std::vector<int64_t> shape(input.sizes().begin(), input.sizes().begin() + axis);
  shape.resize(input.dim(), 1);
  return shape;
}

Tensor contiguous_like(const Tensor& t) {
  return at::empty_like(t, t.options(), at::MemoryFormat::Contiguous);
}

// gamma/beta may be the row dtype, or float32 next to 16-bit rows.
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

}  // namespace

// ---- kernel-entry level ----------------------------------------------------

// layer_norm_kernel, LayerNormKernels.cpp:1418-1438 in the reference.
void layer_norm_kernel(const Tensor& X, const Tensor& gamma, const Tensor& beta, int64_t M,
                       int64_t N, double eps, Tensor* Y, Tensor* mean, Tensor* rstd) {
  static const char* op = "mi355x::layer_norm_kernel";
  check_gpu(X, op, "X");
  TORCH_CHECK(Y != nullptr && Y->defined(), op, ": Y must be allocated by the caller");
  TORCH_CHECK(X.is_contiguous() && Y->is_contiguous(), op, ": X and Y must be contiguous");
  TORCH_CHECK(X.numel() == M * N && Y->numel() == M * N, op, ": X/Y do not hold M*N elements");
  if (mean && mean->defined()) {
    TORCH_CHECK(mean->scalar_type() == at::kFloat && mean->numel() == M, op,
                ": mean must be float32 [M]");
  }
  if (rstd && rstd->defined()) {
    TORCH_CHECK(rstd->scalar_type() == at::kFloat && rstd->numel() == M, op,
                ": rstd must be float32 [M]");
  }
  const rownorm_dtype xd = to_rownorm_dtype(X.scalar_type(), op);
  const rownorm_dtype wd = weight_dtype(X, gamma, beta, op);
  c10::DeviceGuard guard(X.device());
  check_status(mi355x_layer_norm_fwd(X.const_data_ptr(), ptr_or_null(gamma), ptr_or_null(beta),
                                     Y->mutable_data_ptr(), (float*)mut_ptr_or_null(mean),
                                     (float*)mut_ptr_or_null(rstd), M, N, (float)eps, xd, wd,
                                     current_stream(X)),
               op);
}

// rms_norm_kernel, LayerNormKernels.cpp:1465-1491.
void rms_norm_kernel(const Tensor& X, const Tensor& gamma, int64_t M, int64_t N, double eps,
                     Tensor* Y, Tensor* rstd) {
  static const char* op = "mi355x::rms_norm_kernel";
  check_gpu(X, op, "X");
  TORCH_CHECK(Y != nullptr && Y->defined(), op, ": Y must be allocated by the caller");
  TORCH_CHECK(X.is_contiguous() && Y->is_contiguous(), op, ": X and Y must be contiguous");
  TORCH_CHECK(X.numel() == M * N && Y->numel() == M * N, op, ": X/Y do not hold M*N elements");
  if (rstd && rstd->defined()) {
    TORCH_CHECK(rstd->scalar_type() == at::kFloat && rstd->numel() == M, op,
                ": rstd must be float32 [M]");
  }
  const rownorm_dtype xd = to_rownorm_dtype(X.scalar_type(), op);
  const rownorm_dtype wd = weight_dtype(X, gamma, Tensor(), op);
  c10::DeviceGuard guard(X.device());
  check_status(mi355x_rms_norm_fwd(X.const_data_ptr(), ptr_or_null(gamma), Y->mutable_data_ptr(),
                                   (float*)mut_ptr_or_null(rstd), M, N, (float)eps, xd, wd,
                                   current_stream(X)),
               op);
}

// layer_norm_backward_kernel, LayerNormKernels.cpp:1440-1463: dY is made
// contiguous here (:1460); undefined dX/dgamma/dbeta are skipped.
void layer_norm_backward_kernel(const Tensor& dY, const Tensor& X, const Tensor& mean,
                                const Tensor& rstd, const Tensor& gamma, int64_t M, int64_t N,
                                Tensor* dX, Tensor* dgamma, Tensor* dbeta) {
  static const char* op = "mi355x::layer_norm_backward_kernel";
  check_gpu(X, op, "X");
  check_same_device(X, dY, op, "dY");
  TORCH_CHECK(dY.scalar_type() == X.scalar_type(), op, ": dY dtype ", dY.scalar_type(),
              " differs from X dtype ", X.scalar_type());
  TORCH_CHECK(mean.scalar_type() == at::kFloat && rstd.scalar_type() == at::kFloat, op,
              ": mean and rstd must be float32 (the accumulate type), got ", mean.scalar_type(),
              " and ", rstd.scalar_type());
  TORCH_CHECK(mean.numel() == M && rstd.numel() == M && X.numel() == M * N &&
                  dY.numel() == M * N,
              op, ": operand sizes do not match M, N");
  const Tensor dYc = dY.contiguous();
  const Tensor Xc = X.contiguous();
  const Tensor mc = mean.contiguous();
  const Tensor rc = rstd.contiguous();
  void* dx_p = mut_ptr_or_null(dX);
  void* dg_p = mut_ptr_or_null(dgamma);
  void* db_p = mut_ptr_or_null(dbeta);
  if (dx_p) {
    TORCH_CHECK(dX->is_contiguous() && dX->scalar_type() == X.scalar_type() &&
                    dX->numel() == M * N,
                op, ": dX must be a contiguous tensor of the input dtype and size");
  }
  const rownorm_dtype xd = to_rownorm_dtype(X.scalar_type(), op);
  rownorm_dtype wd = xd;
  if (gamma.defined()) wd = weight_dtype(X, gamma, Tensor(), op);
  else if (dg_p) wd = to_rownorm_dtype(dgamma->scalar_type(), op);
  else if (db_p) wd = to_rownorm_dtype(dbeta->scalar_type(), op);
  if (dg_p) {
    TORCH_CHECK(to_rownorm_dtype(dgamma->scalar_type(), op) == wd && dgamma->is_contiguous() &&
                    dgamma->numel() == N,
                op, ": dgamma must be a contiguous [N] tensor of the weight dtype");
  }
  if (db_p) {
    TORCH_CHECK(to_rownorm_dtype(dbeta->scalar_type(), op) == wd && dbeta->is_contiguous() &&
                    dbeta->numel() == N,
                op, ": dbeta must be a contiguous [N] tensor of the weight dtype");
  }
  c10::DeviceGuard guard(X.device());
  const size_t ws_bytes =
      mi355x_layer_norm_bwd_workspace_bytes(M, N, xd, wd, dg_p != nullptr, db_p != nullptr);
  Tensor ws;
  if (ws_bytes > 0) ws = at::empty({(int64_t)ws_bytes}, X.options().dtype(at::kByte));
  check_status(mi355x_layer_norm_bwd(dYc.const_data_ptr(), Xc.const_data_ptr(),
                                     (const float*)mc.const_data_ptr(),
                                     (const float*)rc.const_data_ptr(), ptr_or_null(gamma), dx_p,
                                     dg_p, db_p, ws.defined() ? ws.mutable_data_ptr() : nullptr,
                                     ws_bytes, M, N, xd, wd, current_stream(X)),
               op);
}

// rms_norm_backward_kernel, LayerNormKernels.cpp:1493-1522.
void rms_norm_backward_kernel(const Tensor& dY, const Tensor& X, const Tensor& rstd,
                              const Tensor& gamma, int64_t M, int64_t N, Tensor* dX,
                              Tensor* dgamma) {
  static const char* op = "mi355x::rms_norm_backward_kernel";
  check_gpu(X, op, "X");
  check_same_device(X, dY, op, "dY");
  TORCH_CHECK(dY.scalar_type() == X.scalar_type(), op, ": dY dtype ", dY.scalar_type(),
              " differs from X dtype ", X.scalar_type());
  TORCH_CHECK(rstd.scalar_type() == at::kFloat, op, ": rstd must be float32, got ",
              rstd.scalar_type());
  TORCH_CHECK(rstd.numel() == M && X.numel() == M * N && dY.numel() == M * N, op,
              ": operand sizes do not match M, N");
  const Tensor dYc = dY.contiguous();
  const Tensor Xc = X.contiguous();
  const Tensor rc = rstd.contiguous();
  void* dx_p = mut_ptr_or_null(dX);
  void* dg_p = mut_ptr_or_null(dgamma);
  if (dx_p) {
    TORCH_CHECK(dX->is_contiguous() && dX->scalar_type() == X.scalar_type() &&
                    dX->numel() == M * N,
                op, ": dX must be a contiguous tensor of the input dtype and size");
  }
  const rownorm_dtype xd = to_rownorm_dtype(X.scalar_type(), op);
  rownorm_dtype wd = xd;
  if (gamma.defined()) wd = weight_dtype(X, gamma, Tensor(), op);
  else if (dg_p) wd = to_rownorm_dtype(dgamma->scalar_type(), op);
  if (dg_p) {
    TORCH_CHECK(to_rownorm_dtype(dgamma->scalar_type(), op) == wd && dgamma->is_contiguous() &&
                    dgamma->numel() == N,
                op, ": dgamma must be a contiguous [N] tensor of the weight dtype");
  }
  c10::DeviceGuard guard(X.device());
  const size_t ws_bytes = mi355x_rms_norm_bwd_workspace_bytes(M, N, xd, wd, dg_p != nullptr);
  Tensor ws;
  if (ws_bytes > 0) ws = at::empty({(int64_t)ws_bytes}, X.options().dtype(at::kByte));
  check_status(mi355x_rms_norm_bwd(dYc.const_data_ptr(), Xc.const_data_ptr(),
                                   (const float*)rc.const_data_ptr(), ptr_or_null(gamma), dx_p,
                                   dg_p, ws.defined() ? ws.mutable_data_ptr() : nullptr, ws_bytes,
                                   M, N, xd, wd, current_stream(X)),
               op);
}

// ---- operator level ----------------------------------------------------------

// native_layer_norm: LayerNorm.cpp:35-97.  Y is a contiguous tensor like the
// input; mean and rstd are float32 whatever the input dtype (:72-75) and come
// back shaped input.shape[:axis] + [1]*k (:82-94); nothing is launched when
// M == 0 (:77).
std::tuple<Tensor, Tensor, Tensor> native_layer_norm(const Tensor& input,
                                                     at::IntArrayRef normalized_shape,
                                                     const std::optional<Tensor>& weight_opt,
                                                     const std::optional<Tensor>& bias_opt,
                                                     double epsilon) {
  static const char* op = "mi355x::native_layer_norm";
  if (delegated_dtype(input)) {
    warn_delegated(op);
    return at::cuda::native_layer_norm(input, normalized_shape, weight_opt, bias_opt, epsilon);
  }
  const Tensor weight = defined_or_empty(weight_opt);
  const Tensor bias = defined_or_empty(bias_opt);
  check_same_device(input, weight, op, "weight");
  check_same_device(input, bias, op, "bias");
  const auto [M, N] = at::native::_check_layer_norm_inputs(input, normalized_shape, weight, bias);
  check_gpu(input, op, "input");
  (void)to_rownorm_dtype(input.scalar_type(), op);
  c10::DeviceGuard guard(input.device());
  const Tensor X = input.contiguous();
  const Tensor gamma = weight.defined() ? weight.contiguous() : weight;
  const Tensor beta = bias.defined() ? bias.contiguous() : bias;
  Tensor Y = contiguous_like(X);
  Tensor mean = at::empty({M}, X.options().dtype(at::kFloat));
  Tensor rstd = at::empty({M}, X.options().dtype(at::kFloat));
  if (M > 0 && N > 0) {
    layer_norm_kernel(X, gamma, beta, M, N, epsilon, &Y, &mean, &rstd);
  } else if (M > 0) {
    // rows of no elements: what the CPU kernel's formulas give, mean 0 and rstd NaN
    mean.zero_();
    rstd.fill_(std::numeric_limits<float>::quiet_NaN());
  }
  const auto stat_shape = stat_shape_of(input, normalized_shape.size());
  return std::make_tuple(std::move(Y), mean.view(stat_shape), rstd.view(stat_shape));
}

// native_layer_norm_backward: LayerNorm.cpp:99-196.  Only the outputs whose
// mask bit is set are allocated, the rest stay undefined; dgamma/dbeta are
// zeros when M == 0 (:150-181).
std::tuple<Tensor, Tensor, Tensor> native_layer_norm_backward(
    const Tensor& grad_output, const Tensor& input, at::IntArrayRef normalized_shape,
    const Tensor& mean, const Tensor& rstd, const std::optional<Tensor>& weight_opt,
    const std::optional<Tensor>& bias_opt, std::array<bool, 3> grad_input_mask) {
  static const char* op = "mi355x::native_layer_norm_backward";
  if (delegated_dtype(input)) {
    warn_delegated(op);
    return at::cuda::native_layer_norm_backward(grad_output, input, normalized_shape, mean, rstd,
                                                weight_opt, bias_opt, grad_input_mask);
  }
  const Tensor weight = defined_or_empty(weight_opt);
  const Tensor bias = defined_or_empty(bias_opt);
  check_same_device(input, grad_output, op, "grad_out");
  check_same_device(input, mean, op, "mean");
  check_same_device(input, rstd, op, "rstd");
  check_same_device(input, weight, op, "weight");
  check_same_device(input, bias, op, "bias");
  const auto [M, N] = at::native::_check_layer_norm_inputs(input, normalized_shape, weight, bias);
  check_gpu(input, op, "input");
  (void)to_rownorm_dtype(input.scalar_type(), op);
  c10::DeviceGuard guard(input.device());
  const Tensor X = input.contiguous();
  const Tensor gamma = weight.defined() ? weight.contiguous() : weight;
  const Tensor beta = bias.defined() ? bias.contiguous() : bias;

  Tensor dX, dgamma, dbeta;
  if (grad_input_mask[0]) dX = contiguous_like(X);
  if (grad_input_mask[1] && gamma.defined())
    dgamma = M > 0 ? contiguous_like(gamma) : at::zeros_like(gamma, at::MemoryFormat::Contiguous);
  if (grad_input_mask[2] && beta.defined())
    dbeta = M > 0 ? contiguous_like(beta) : at::zeros_like(beta, at::MemoryFormat::Contiguous);
  if (M > 0 && N > 0)
    layer_norm_backward_kernel(grad_output, X, mean, rstd, gamma, M, N, &dX, &dgamma, &dbeta);
  return std::make_tuple(std::move(dX), std::move(dgamma), std::move(dbeta));
}

// _fused_rms_norm: LayerNorm.cpp:203-253.  eps defaults to FLT_EPSILON, the
// epsilon of the float32 accumulate type (:218-224); returns (Y, rstd).
std::tuple<Tensor, Tensor> _fused_rms_norm(const Tensor& input, at::IntArrayRef normalized_shape,
                                           const std::optional<Tensor>& weight_opt,
                                           std::optional<double> eps_opt) {
  static const char* op = "mi355x::_fused_rms_norm";
  if (delegated_dtype(input)) {
    warn_delegated(op);
    return at::cuda::_fused_rms_norm(input, normalized_shape, weight_opt, eps_opt);
  }
  const Tensor weight = defined_or_empty(weight_opt);
  check_same_device(input, weight, op, "weight");
  const auto [M, N] =
      at::native::_check_layer_norm_inputs(input, normalized_shape, weight, weight);
  check_gpu(input, op, "input");
  (void)to_rownorm_dtype(input.scalar_type(), op);
  c10::DeviceGuard guard(input.device());
  const Tensor X = input.contiguous();
  const Tensor gamma = weight.defined() ? weight.contiguous() : weight;
  const double eps = eps_opt.value_or((double)std::numeric_limits<float>::epsilon());
  Tensor Y = contiguous_like(X);
  Tensor rstd = at::empty({M}, X.options().dtype(at::kFloat));
  if (M > 0 && N > 0) {
    rms_norm_kernel(X, gamma, M, N, eps, &Y, &rstd);
  } else if (M > 0) {
    rstd.fill_(std::numeric_limits<float>::quiet_NaN());  // the mean of no squares, as on the CPU
  }
  return std::make_tuple(std::move(Y), rstd.view(stat_shape_of(input, normalized_shape.size())));
}

// _fused_rms_norm_backward: LayerNorm.cpp:255-305.
std::tuple<Tensor, Tensor> _fused_rms_norm_backward(const Tensor& dY, const Tensor& input,
                                                    at::IntArrayRef normalized_shape,
                                                    const Tensor& rstd,
                                                    const std::optional<Tensor>& weight_opt,
                                                    std::array<bool, 2> grad_input_mask) {
  static const char* op = "mi355x::_fused_rms_norm_backward";
  if (delegated_dtype(input)) {
    warn_delegated(op);
    return at::cuda::_fused_rms_norm_backward(dY, input, normalized_shape, rstd, weight_opt,
                                              grad_input_mask);
  }
  const Tensor weight = defined_or_empty(weight_opt);
  check_same_device(input, dY, op, "grad_out");
  check_same_device(input, rstd, op, "rstd");
  check_same_device(input, weight, op, "weight");
  const auto [M, N] =
      at::native::_check_layer_norm_inputs(input, normalized_shape, weight, weight);
  check_gpu(input, op, "input");
  (void)to_rownorm_dtype(input.scalar_type(), op);
  c10::DeviceGuard guard(input.device());
  const Tensor X = input.contiguous();
  const Tensor gamma = weight.defined() ? weight.contiguous() : weight;
  Tensor dX, dgamma;
  if (grad_input_mask[0]) dX = contiguous_like(X);
  if (grad_input_mask[1] && gamma.defined())
    dgamma = M > 0 ? contiguous_like(gamma) : at::zeros_like(gamma, at::MemoryFormat::Contiguous);
  if (M > 0 && N > 0) rms_norm_backward_kernel(dY, X, rstd, gamma, M, N, &dX, &dgamma);
  return std::make_tuple(std::move(dX), std::move(dgamma));
}

// ---- ATen dispatch stubs -------------------------------------------------------

namespace {

struct SavedStubs {
  bool installed = false;
  void* forward = nullptr;
  void* backward = nullptr;
};
SavedStubs g_layer_norm_saved;

void stub_forward(const Tensor& X, const Tensor& gamma, const Tensor& beta, int64_t M, int64_t N,
                  double eps, Tensor* Y, Tensor* mean, Tensor* rstd) {
  if (delegated_dtype(X) && g_layer_norm_saved.forward != nullptr) {
    warn_delegated("LayerNormKernel");
    return reinterpret_cast<at::native::forward_fn>(g_layer_norm_saved.forward)(
        X, gamma, beta, M, N, eps, Y, mean, rstd);
  }
  layer_norm_kernel(X, gamma, beta, M, N, eps, Y, mean, rstd);
}
void stub_backward(const Tensor& dY, const Tensor& X, const Tensor& mean, const Tensor& rstd,
                   const Tensor& gamma, int64_t M, int64_t N, Tensor* dX, Tensor* dgamma,
                   Tensor* dbeta) {
  if (delegated_dtype(X) && g_layer_norm_saved.backward != nullptr) {
    warn_delegated("LayerNormBackwardKernel");
    return reinterpret_cast<at::native::backward_fn>(g_layer_norm_saved.backward)(
        dY, X, mean, rstd, gamma, M, N, dX, dgamma, dbeta);
  }
  layer_norm_backward_kernel(dY, X, mean, rstd, gamma, M, N, dX, dgamma, dbeta);
}
}  // namespace

void install_layer_norm_dispatch_stubs() {
  if (g_layer_norm_saved.installed) return;
  g_layer_norm_saved.forward =
      install_checked(at::native::LayerNormKernel, &stub_forward, "LayerNormKernel");
  g_layer_norm_saved.backward = install_checked(at::native::LayerNormBackwardKernel,
                                                &stub_backward, "LayerNormBackwardKernel");
  g_layer_norm_saved.installed = true;
}

void uninstall_layer_norm_dispatch_stubs() {
  if (!g_layer_norm_saved.installed) return;
  restore<decltype(at::native::LayerNormKernel), std::remove_pointer_t<at::native::forward_fn>>(
      at::native::LayerNormKernel, g_layer_norm_saved.forward);
  restore<decltype(at::native::LayerNormBackwardKernel),
          std::remove_pointer_t<at::native::backward_fn>>(at::native::LayerNormBackwardKernel,
                                                          g_layer_norm_saved.backward);
  g_layer_norm_saved = SavedStubs{};
}

}  // namespace mi355x
