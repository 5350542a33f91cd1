// Host dispatch of the non-innermost-dimension softmax kernels: plan -> template instance.
#pragma once
#include "launch.hpp"
#include "softmax_strided_kernels.hpp"

namespace rownorm {

template <class TI, class TO, int V, bool FAST>
void launch_strided_fwd_v(const StridedPlan& p, const SoftmaxStridedFwdArgs& a, hipStream_t s) {
  hipLaunchKernelGGL((softmax_strided_fwd_kernel<TI, TO, V, kStridedBlock, FAST>),
                     dim3((unsigned)p.grid), dim3(kStridedBlock), 0, s, (const TI*)a.x, (TO*)a.y,
                     a.outer, a.D, a.inner, StridedLayout{p.tx_log2, p.ty_log2}, a.flags);
}

template <class TI, class TO, bool FAST>
bool launch_strided_fwd_f(const StridedPlan& p, const SoftmaxStridedFwdArgs& a, hipStream_t s) {
  switch (p.V) {
    case 1: launch_strided_fwd_v<TI, TO, 1, FAST>(p, a, s); return true;
    case 2: launch_strided_fwd_v<TI, TO, 2, FAST>(p, a, s); return true;
    case 3: launch_strided_fwd_v<TI, TO, 3, FAST>(p, a, s); return true;
    case 4: launch_strided_fwd_v<TI, TO, 4, FAST>(p, a, s); return true;
    case 5: launch_strided_fwd_v<TI, TO, 5, FAST>(p, a, s); return true;
    case 6: launch_strided_fwd_v<TI, TO, 6, FAST>(p, a, s); return true;
    case 7: launch_strided_fwd_v<TI, TO, 7, FAST>(p, a, s); return true;
    case 8: launch_strided_fwd_v<TI, TO, 8, FAST>(p, a, s); return true;
  }
  return false;
}

template <class TI, class TO>
int launch_softmax_strided_fwd(const StridedPlan& p, const SoftmaxStridedFwdArgs& a,
                               hipStream_t s) {
  if (p.resident) {
    const bool ok = p.fast ? launch_strided_fwd_f<TI, TO, true>(p, a, s)
                           : launch_strided_fwd_f<TI, TO, false>(p, a, s);
    if (!ok) return (int)hipErrorInvalidConfiguration;
  } else {
    hipLaunchKernelGGL((softmax_strided_fwd_stream_kernel<TI, TO, kStridedBlock>),
                       dim3((unsigned)p.grid), dim3(kStridedBlock), 0, s, (const TI*)a.x,
                       (TO*)a.y, a.outer, a.D, a.inner, StridedLayout{p.tx_log2, p.ty_log2},
                       a.flags);
  }
  return (int)hipGetLastError();
}

template <class TG, class TO, int V, bool FAST>
void launch_strided_bwd_v(const StridedPlan& p, const SoftmaxStridedBwdArgs& a, hipStream_t s) {
  hipLaunchKernelGGL((softmax_strided_bwd_kernel<TG, TO, V, kStridedBlock, FAST>),
                     dim3((unsigned)p.grid), dim3(kStridedBlock), 0, s, (const TG*)a.grad,
                     (const TG*)a.y, (TO*)a.gi, a.outer, a.D, a.inner,
                     StridedLayout{p.tx_log2, p.ty_log2}, a.flags);
}

template <class TG, class TO, bool FAST>
bool launch_strided_bwd_f(const StridedPlan& p, const SoftmaxStridedBwdArgs& a, hipStream_t s) {
  switch (p.V) {
    case 1: launch_strided_bwd_v<TG, TO, 1, FAST>(p, a, s); return true;
    case 2: launch_strided_bwd_v<TG, TO, 2, FAST>(p, a, s); return true;
    case 3: launch_strided_bwd_v<TG, TO, 3, FAST>(p, a, s); return true;
    case 4: launch_strided_bwd_v<TG, TO, 4, FAST>(p, a, s); return true;
    case 5: launch_strided_bwd_v<TG, TO, 5, FAST>(p, a, s); return true;
    case 6: launch_strided_bwd_v<TG, TO, 6, FAST>(p, a, s); return true;
    case 7: launch_strided_bwd_v<TG, TO, 7, FAST>(p, a, s); return true;
    case 8: launch_strided_bwd_v<TG, TO, 8, FAST>(p, a, s); return true;
  }
  return false;
}

template <class TG, class TO>
int launch_softmax_strided_bwd(const StridedPlan& p, const SoftmaxStridedBwdArgs& a,
                               hipStream_t s) {
  if (p.resident) {
    const bool ok = p.fast ? launch_strided_bwd_f<TG, TO, true>(p, a, s)
                           : launch_strided_bwd_f<TG, TO, false>(p, a, s);
    if (!ok) return (int)hipErrorInvalidConfiguration;
  } else {
    hipLaunchKernelGGL((softmax_strided_bwd_stream_kernel<TG, TO, kStridedBlock>),
                       dim3((unsigned)p.grid), dim3(kStridedBlock), 0, s, (const TG*)a.grad,
                       (const TG*)a.y, (TO*)a.gi, a.outer, a.D, a.inner,
                     StridedLayout{p.tx_log2, p.ty_log2}, a.flags);
  }
  return (int)hipGetLastError();
}

}  // namespace rownorm
