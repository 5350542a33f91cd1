// Shared helpers of the ATen-facing host layer: dtype mapping, stream lookup,
// error translation.  The host layer owns argument validation, contiguity,
// output and workspace allocation (through ATen's caching allocator) and the
// current-stream lookup; the kernels behind include/mi355x_rownorm.h own
// nothing.  There is no CPU path: a tensor that is not on a GPU is an error.
#pragma once
#include <ATen/ATen.h>
#include <c10/hip/HIPStream.h>
#include <c10/core/DeviceGuard.h>

#include "mi355x_rownorm.h"

namespace mi355x {

inline rownorm_dtype to_rownorm_dtype(at::ScalarType t, const char* op) {
  switch (t) {
    case at::kFloat: return ROWNORM_F32;
    case at::kHalf: return ROWNORM_F16;
    case at::kBFloat16: return ROWNORM_BF16;
    default:
      TORCH_CHECK(false, op, ": dtype ", t,
                  " is not implemented by the MI355X kernels (float32, float16 and bfloat16 are)");
  }
}

// float64 is outside what the MI355X kernels compute (float32 accumulation): the
// operator level hands such calls to the kernels PyTorch-ROCm itself ships, with
// one warning per process, in the way the reference hands what it lacks to
// another backend (src/ATen/native/xpu/XPUFallback.cpp:59-69).  The reference
// itself accumulates float64 in double (sycl/LayerNormKernels.cpp:1418-1438).
inline bool delegated_dtype(const at::Tensor& t) {
  return t.defined() && t.is_cuda() && t.scalar_type() == at::kDouble;
}

inline void warn_delegated(const char* op) {
  TORCH_WARN_ONCE("mi355x: float64 tensors are delegated to the stock PyTorch-ROCm kernels (first "
                  "seen in ", op, "); the MI355X kernels compute float32, float16 and bfloat16");
}

inline void check_gpu(const at::Tensor& t, const char* op, const char* name) {
  TORCH_CHECK(t.is_cuda(), op, ": expected `", name,
              "` on a HIP GPU device, but it is on ", t.device(),
              " (this library has no CPU path)");
}

inline void check_same_device(const at::Tensor& ref, const at::Tensor& t, const char* op,
                              const char* name) {
  if (t.defined()) {
    TORCH_CHECK(t.device() == ref.device(), op, ": expected `", name, "` on ", ref.device(),
                " like the input, but it is on ", t.device());
  }
}

inline void* current_stream(const at::Tensor& t) {
  return (void*)c10::hip::getCurrentHIPStream(t.device().index()).stream();
}

inline void check_status(int code, const char* op) {
  TORCH_CHECK(code == 0, op, ": ", mi355x_rownorm_error_string(code), " (code ", code, ")");
}

inline const void* ptr_or_null(const at::Tensor& t) {
  return t.defined() ? t.const_data_ptr() : nullptr;
}
inline void* mut_ptr_or_null(at::Tensor* t) {
  return (t != nullptr && t->defined()) ? t->mutable_data_ptr() : nullptr;
}

}  // namespace mi355x
