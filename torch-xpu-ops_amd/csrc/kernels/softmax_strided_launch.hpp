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
  } else if (p.chunks > 1 &&
             regions_disjoint(a.y, a.outer * (int64_t)a.D * a.inner * (int64_t)sizeof(TO), a.x,
                              a.outer * (int64_t)a.D * a.inner * (int64_t)sizeof(TI))) {
    // the D rows of a tile are split over workgroups; the per-column values cross the
    // three launches inside y, which therefore must not be x
    constexpr int E = elems_per_pack<TI>::value;
    const StridedLayout lay{p.tx_log2, p.ty_log2};
    const dim3 grid((unsigned)p.grid, (unsigned)p.chunks);
    hipLaunchKernelGGL((softmax_strided_split_partial_kernel<TI, TO, kStridedBlock>), grid,
                       dim3(kStridedBlock), 0, s, (const TI*)a.x, (TO*)a.y, a.outer, a.D, a.inner,
                       lay, p.chunk_rows);
    hipLaunchKernelGGL((softmax_strided_split_combine_kernel<TO, E, 2, kStridedBlock>),
                       dim3((unsigned)p.grid), dim3(kStridedBlock), 0, s, (TO*)a.y, a.outer, a.D,
                       a.inner, lay, p.chunk_rows, p.chunks);
    hipLaunchKernelGGL((softmax_strided_split_apply_kernel<TI, TO, kStridedBlock>), grid,
                       dim3(kStridedBlock), 0, s, (const TI*)a.x, (TO*)a.y, a.outer, a.D, a.inner,
                       lay, p.chunk_rows, a.flags);
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
  } else if (p.chunks > 1 && [&] {
               const int64_t n = a.outer * (int64_t)a.D * a.inner;
               const int64_t ob = n * (int64_t)sizeof(TO), ib = n * (int64_t)sizeof(TG);
               return regions_disjoint(a.gi, ob, a.grad, ib) && regions_disjoint(a.gi, ob, a.y, ib);
             }()) {
    constexpr int E = elems_per_pack<TG>::value;
    const StridedLayout lay{p.tx_log2, p.ty_log2};
    const dim3 grid((unsigned)p.grid, (unsigned)p.chunks);
    hipLaunchKernelGGL((softmax_strided_split_bwd_partial_kernel<TG, TO, kStridedBlock>), grid,
                       dim3(kStridedBlock), 0, s, (const TG*)a.grad, (const TG*)a.y, (TO*)a.gi,
                       a.outer, a.D, a.inner, lay, p.chunk_rows, a.flags);
    hipLaunchKernelGGL((softmax_strided_split_combine_kernel<TO, E, 1, kStridedBlock>),
                       dim3((unsigned)p.grid), dim3(kStridedBlock), 0, s, (TO*)a.gi, a.outer, a.D,
                       a.inner, lay, p.chunk_rows, p.chunks);
    hipLaunchKernelGGL((softmax_strided_split_bwd_apply_kernel<TG, TO, kStridedBlock>), grid,
                       dim3(kStridedBlock), 0, s, (const TG*)a.grad, (const TG*)a.y, (TO*)a.gi,
                       a.outer, a.D, a.inner, lay, p.chunk_rows, a.flags);
  } else {
    hipLaunchKernelGGL((softmax_strided_bwd_stream_kernel<TG, TO, kStridedBlock>),
                       dim3((unsigned)p.grid), dim3(kStridedBlock), 0, s, (const TG*)a.grad,
                       (const TG*)a.y, (TO*)a.gi, a.outer, a.D, a.inner,
                     StridedLayout{p.tx_log2, p.ty_log2}, a.flags);
  }
  return (int)hipGetLastError();
}

}  // namespace rownorm
