// GroupNorm host operators: shape checks, output allocation, then one call into
// the C ABI.  The kernel entries follow the reference's group_norm_kernel /
// group_norm_backward_kernel (src/ATen/native/xpu/sycl/GroupNormKernels.cpp:
// 364-530, 1353-1589); the operator level restates ATen's native_group_norm
// host function, which the reference inherits from upstream.
#include "group_norm_ops.h"

#include <ATen/native/group_norm.h>
#include <ATen/ops/native_group_norm_backward_cuda_dispatch.h>
#include <ATen/ops/native_group_norm_cuda_dispatch.h>
#include <limits>

#include "dispatch_stub_slot.h"
#include "host_common.h"

namespace mi355x {
namespace {

using at::Tensor;

Tensor defined_or_empty(const std::optional<Tensor>& t) {
  return (t.has_value() && t->defined()) ? *t : Tensor();
}

// The statistics dtype: float32 beside float32 weights of a 16-bit input,
// otherwise the input dtype (what ATen's param_scalar_type gives).
rownorm_dtype stat_dtype(const Tensor& X, const Tensor& gamma, const Tensor& beta,
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

at::ScalarType to_scalar_type(rownorm_dtype d) {
  return d == ROWNORM_F32 ? at::kFloat : d == ROWNORM_F16 ? at::kHalf : at::kBFloat16;
}

struct SavedStubs {
  bool installed = false;
  void* forward = nullptr;
  void* backward = nullptr;
};
SavedStubs g_group_norm_saved;

}  // namespace

// group_norm_kernel, GroupNormKernels.cpp:499-530 (checks at :377-379).
void group_norm_kernel(const Tensor& X, const Tensor& gamma, const Tensor& beta, int64_t N,
                       int64_t C, int64_t HxW, int64_t group, double eps, Tensor& Y, Tensor& mean,
                       Tensor& rstd) {
  static const char* op = "mi355x::group_norm_kernel";
  if (delegated_dtype(X) && g_group_norm_saved.forward != nullptr) {
    // reached through ATen's GroupNormKernel stub: pass float64 on to the kernel
    // that was registered before
    warn_delegated(op);
    return reinterpret_cast<at::native::forward_fn>(g_group_norm_saved.forward)(
        X, gamma, beta, N, C, HxW, group, eps, Y, mean, rstd);
  }
  check_gpu(X, op, "X");
  TORCH_CHECK(X.numel() == N * C * HxW, op, ": X does not hold N*C*HxW elements");
  TORCH_CHECK(!gamma.defined() || gamma.numel() == C, op, ": gamma must hold C elements");
  TORCH_CHECK(!beta.defined() || beta.numel() == C, op, ": beta must hold C elements");
  TORCH_CHECK(Y.defined() && Y.is_contiguous() && Y.numel() == X.numel() &&
                  Y.scalar_type() == X.scalar_type(),
              op, ": Y must be a contiguous tensor of the input dtype and size");
  if (N == 0) return;
  const rownorm_dtype xd = to_rownorm_dtype(X.scalar_type(), op);
  const rownorm_dtype sd = stat_dtype(X, gamma, beta, op);
  if (C == 0 || HxW == 0) {
    // groups of no elements: what the CPU kernel's formulas give, mean 0 and rstd NaN
    if (mean.defined()) mean.zero_();
    if (rstd.defined()) rstd.fill_(std::numeric_limits<double>::quiet_NaN());
    return;
  }
  for (const Tensor* t : {&mean, &rstd}) {
    if (t->defined()) {
      TORCH_CHECK(t->is_contiguous() && t->numel() == N * group &&
                      t->scalar_type() == to_scalar_type(sd),
                  op, ": mean and rstd must be contiguous [N, group] tensors of dtype ",
                  to_scalar_type(sd));
    }
  }
  const Tensor Xc = X.contiguous();
  const Tensor gc = gamma.defined() ? gamma.contiguous() : gamma;
  const Tensor bc = beta.defined() ? beta.contiguous() : beta;
  c10::DeviceGuard guard(X.device());
  check_status(mi355x_group_norm_fwd(Xc.const_data_ptr(), ptr_or_null(gc), ptr_or_null(bc),
                                     Y.mutable_data_ptr(), mut_ptr_or_null(&mean),
                                     mut_ptr_or_null(&rstd), N, C, HxW, group, (float)eps, xd, sd,
                                     current_stream(X)),
               op);
}

// group_norm_backward_kernel, GroupNormKernels.cpp:1565-1589 (checks at
// :1373-1377).  Undefined dX / dgamma / dbeta are skipped.
void group_norm_backward_kernel(const Tensor& dY, const Tensor& X, const Tensor& mean,
                                const Tensor& rstd, const Tensor& gamma, int64_t N, int64_t C,
                                int64_t HxW, int64_t group, Tensor& dX, Tensor& dgamma,
                                Tensor& dbeta) {
  static const char* op = "mi355x::group_norm_backward_kernel";
  if (delegated_dtype(X) && g_group_norm_saved.backward != nullptr) {
    warn_delegated(op);
    return reinterpret_cast<at::native::backward_fn>(g_group_norm_saved.backward)(
        dY, X, mean, rstd, gamma, N, C, HxW, group, dX, dgamma, dbeta);
  }
  check_gpu(X, op, "X");
  check_same_device(X, dY, op, "dY");
  TORCH_CHECK(dY.numel() == N * C * HxW && X.numel() == N * C * HxW, op,
              ": dY and X must hold N*C*HxW elements");
  TORCH_CHECK(mean.numel() == N * group && rstd.numel() == N * group, op,
              ": mean and rstd must hold N*group elements");
  TORCH_CHECK(!gamma.defined() || gamma.numel() == C, op, ": gamma must hold C elements");
  TORCH_CHECK(dY.scalar_type() == X.scalar_type(), op, ": dY dtype ", dY.scalar_type(),
              " differs from X dtype ", X.scalar_type());
  TORCH_CHECK(mean.scalar_type() == rstd.scalar_type(), op, ": mean and rstd must share a dtype");
  const rownorm_dtype xd = to_rownorm_dtype(X.scalar_type(), op);
  const rownorm_dtype sd = to_rownorm_dtype(mean.scalar_type(), op);
  TORCH_CHECK(sd == xd || sd == ROWNORM_F32, op,
              ": mean/rstd dtype must equal the input dtype or be float32, got ",
              mean.scalar_type());
  TORCH_CHECK(!gamma.defined() || to_rownorm_dtype(gamma.scalar_type(), op) == sd, op,
              ": gamma dtype ", gamma.scalar_type(), " must match mean/rstd dtype ",
              mean.scalar_type());
  if (dX.defined()) {
    TORCH_CHECK(dX.is_contiguous() && dX.scalar_type() == X.scalar_type() &&
                    dX.numel() == X.numel(),
                op, ": dX must be a contiguous tensor of the input dtype and size");
  }
  for (const Tensor* t : {&dgamma, &dbeta}) {
    if (t->defined()) {
      TORCH_CHECK(t->is_contiguous() && t->numel() == C &&
                      t->scalar_type() == mean.scalar_type(),
                  op, ": dgamma and dbeta must be contiguous [C] tensors of dtype ",
                  mean.scalar_type());
    }
  }
  if (N == 0 || C == 0 || HxW == 0) {
    if (dgamma.defined()) dgamma.zero_();
    if (dbeta.defined()) dbeta.zero_();
    return;
  }
  const Tensor dYc = dY.contiguous();
  const Tensor Xc = X.contiguous();
  const Tensor mc = mean.contiguous();
  const Tensor rc = rstd.contiguous();
  const Tensor gc = gamma.defined() ? gamma.contiguous() : gamma;
  c10::DeviceGuard guard(X.device());
  const size_t nbytes = mi355x_group_norm_bwd_workspace_bytes(N, C, HxW, group, xd, sd,
                                                              dgamma.defined(), dbeta.defined());
  Tensor workspace;
  if (nbytes > 0) workspace = at::empty({(int64_t)nbytes}, X.options().dtype(at::kByte));
  check_status(
      mi355x_group_norm_bwd(dYc.const_data_ptr(), Xc.const_data_ptr(), mc.const_data_ptr(),
                            rc.const_data_ptr(), ptr_or_null(gc), mut_ptr_or_null(&dX),
                            mut_ptr_or_null(&dgamma), mut_ptr_or_null(&dbeta),
                            mut_ptr_or_null(&workspace), nbytes, N, C, HxW, group, xd, sd,
                            current_stream(X)),
      op);
}

// aten::native_group_norm: argument checks with ATen's messages, contiguous
// NCHW output, statistics [N, group] in the parameter dtype.
std::tuple<Tensor, Tensor, Tensor> native_group_norm(const Tensor& X,
                                                     const std::optional<Tensor>& weight_opt,
                                                     const std::optional<Tensor>& bias_opt,
                                                     int64_t N, int64_t C, int64_t HxW,
                                                     int64_t group, double eps) {
  static const char* op = "mi355x::native_group_norm";
  if (delegated_dtype(X)) {
    warn_delegated(op);
    return at::cuda::native_group_norm(X, weight_opt, bias_opt, N, C, HxW, group, eps);
  }
  const Tensor gamma = defined_or_empty(weight_opt);
  const Tensor beta = defined_or_empty(bias_opt);
  TORCH_CHECK(group > 0, "Expected num groups to be greater than 0, got ", group);
  TORCH_CHECK(C % group == 0,
              "Expected number of channels in input to be divisible by ", "num_groups, but got input of shape ",
              X.sizes(), " and num_groups=", group);
  TORCH_CHECK(!gamma.defined() || (gamma.dim() == 1 && gamma.numel() == C),
              "Expected weight to be a vector of size equal to the number of ",
              "channels in input, but got weight of shape ", gamma.sizes(),
              " and input of shape ", X.sizes());
  TORCH_CHECK(!beta.defined() || (beta.dim() == 1 && beta.numel() == C),
              "Expected bias to be a vector of size equal to the number of ",
              "channels in input, but got bias of shape ", beta.sizes(), " and input of shape ",
              X.sizes());
  TORCH_CHECK(X.numel() == N * C * HxW, op, ": input of shape ", X.sizes(),
              " does not hold N*C*HxW = ", N, "*", C, "*", HxW, " elements");
  check_gpu(X, op, "input");
  check_same_device(X, gamma, op, "weight");
  check_same_device(X, beta, op, "bias");
  const rownorm_dtype sd = stat_dtype(X, gamma, beta, op);
  (void)to_rownorm_dtype(X.scalar_type(), op);
  Tensor Y = at::empty_like(X, X.options(), at::MemoryFormat::Contiguous);
  Tensor mean = at::empty({N, group}, X.options().dtype(to_scalar_type(sd)));
  Tensor rstd = at::empty({N, group}, X.options().dtype(to_scalar_type(sd)));
  group_norm_kernel(X, gamma, beta, N, C, HxW, group, eps, Y, mean, rstd);
  return std::make_tuple(std::move(Y), std::move(mean), std::move(rstd));
}

// aten::native_group_norm_backward: only the gradients whose mask bit is set
// are allocated and computed; the rest come back undefined.
std::tuple<Tensor, Tensor, Tensor> native_group_norm_backward(
    const Tensor& dY, const Tensor& X, const Tensor& mean, const Tensor& rstd,
    const std::optional<Tensor>& weight_opt, int64_t N, int64_t C, int64_t HxW, int64_t group,
    std::array<bool, 3> output_mask) {
  static const char* op = "mi355x::native_group_norm_backward";
  if (delegated_dtype(X)) {
    warn_delegated(op);
    return at::cuda::native_group_norm_backward(dY, X, mean, rstd, weight_opt, N, C, HxW, group,
                                                output_mask);
  }
  const Tensor gamma = defined_or_empty(weight_opt);
  TORCH_CHECK(X.scalar_type() == dY.scalar_type(), "Expected scalar types of X and dY are same.");
  check_gpu(X, op, "input");
  check_same_device(X, dY, op, "grad_out");
  check_same_device(X, mean, op, "mean");
  check_same_device(X, rstd, op, "rstd");
  check_same_device(X, gamma, op, "weight");
  Tensor dX, dgamma, dbeta;
  if (output_mask[0]) dX = at::empty_like(X, X.options(), at::MemoryFormat::Contiguous);
  if (output_mask[1]) dgamma = at::empty({C}, X.options().dtype(mean.scalar_type()));
  if (output_mask[2]) dbeta = at::empty({C}, X.options().dtype(mean.scalar_type()));
  group_norm_backward_kernel(dY, X, mean, rstd, gamma, N, C, HxW, group, dX, dgamma, dbeta);
  return std::make_tuple(std::move(dX), std::move(dgamma), std::move(dbeta));
}

void install_group_norm_dispatch_stubs() {
  if (g_group_norm_saved.installed) return;
  g_group_norm_saved.forward =
      install_checked(at::native::GroupNormKernel, &group_norm_kernel, "GroupNormKernel");
  g_group_norm_saved.backward = install_checked(at::native::GroupNormBackwardKernel,
                                                &group_norm_backward_kernel,
                                                "GroupNormBackwardKernel");
  g_group_norm_saved.installed = true;
}

void uninstall_group_norm_dispatch_stubs() {
  if (!g_group_norm_saved.installed) return;
  restore<decltype(at::native::GroupNormKernel),
          std::remove_pointer_t<at::native::forward_fn>>(at::native::GroupNormKernel,
                                                         g_group_norm_saved.forward);
  restore<decltype(at::native::GroupNormBackwardKernel),
          std::remove_pointer_t<at::native::backward_fn>>(at::native::GroupNormBackwardKernel,
                                                          g_group_norm_saved.backward);
  g_group_norm_saved = SavedStubs{};
}

}  // namespace mi355x
