// Host dispatch of the softmax / log_softmax kernels: plan -> template instance.
#pragma once
#include "launch.hpp"
#include "softmax_kernels.hpp"

namespace rownorm {

template <class TI, class TO>
struct SoftmaxFwdCtx {
  const Plan& plan;
  const SoftmaxFwdArgs& a;
  hipStream_t stream;
};

template <class TI, class TO, bool FAST, bool MASKED>
struct SoftmaxFwdLauncher {
  template <int G, int V, int BLOCK>
  struct At {
    static bool run(const SoftmaxFwdCtx<TI, TO>& c) {
      if constexpr (variant_built(OC_SOFTMAX_FWD, sizeof(TI), G, V, FAST) &&
                    block_built(OC_SOFTMAX_FWD, G, BLOCK)) {
        if (c.plan.G == G && c.plan.V == V && c.plan.block == BLOCK) {
          hipLaunchKernelGGL((softmax_fwd_resident_kernel<TI, TO, G, V, BLOCK, FAST, MASKED>),
                             dim3((unsigned)c.plan.grid), dim3(BLOCK), 0, c.stream,
                             (const TI*)c.a.x, (TO*)c.a.y,
                             MaskRef{c.a.mask, c.a.mask_div, c.a.mask_mod, c.a.mask_stride}, c.a.M, c.a.N,
                             c.a.flags);
          return true;
        }
      }
      return false;
    }
  };
};

template <class TI, class TO, bool MASKED>
int launch_softmax_fwd_m(const Plan& plan, const SoftmaxFwdArgs& a, hipStream_t stream) {
  if (plan.resident) {
    SoftmaxFwdCtx<TI, TO> ctx{plan, a, stream};
    const bool launched =
        plan.fast ? launch_variant<SoftmaxFwdLauncher<TI, TO, true, MASKED>::template At>(ctx)
                  : launch_variant<SoftmaxFwdLauncher<TI, TO, false, MASKED>::template At>(ctx);
    if (!launched) return (int)hipErrorInvalidConfiguration;
  } else {
    hipLaunchKernelGGL((softmax_fwd_stream_kernel<TI, TO, kStreamBlock, MASKED>),
                       dim3((unsigned)plan.grid), dim3(kStreamBlock), 0, stream, (const TI*)a.x,
                       (TO*)a.y, MaskRef{a.mask, a.mask_div, a.mask_mod, a.mask_stride}, a.M, a.N, a.flags);
  }
  return (int)hipGetLastError();
}

template <class TI, class TO>
int launch_softmax_fwd(const Plan& plan, const SoftmaxFwdArgs& a, hipStream_t stream) {
  return a.mask ? launch_softmax_fwd_m<TI, TO, true>(plan, a, stream)
                : launch_softmax_fwd_m<TI, TO, false>(plan, a, stream);
}

template <class TG, class TO>
struct SoftmaxBwdCtx {
  const Plan& plan;
  const SoftmaxBwdArgs& a;
  hipStream_t stream;
};

template <class TG, class TO, bool FAST, bool MASKED>
struct SoftmaxBwdLauncher {
  template <int G, int V, int BLOCK>
  struct At {
    static bool run(const SoftmaxBwdCtx<TG, TO>& c) {
      if constexpr (variant_built(OC_SOFTMAX_BWD, sizeof(TG), G, V, FAST) &&
                    block_built(OC_SOFTMAX_BWD, G, BLOCK)) {
        if (c.plan.G == G && c.plan.V == V && c.plan.block == BLOCK) {
          hipLaunchKernelGGL((softmax_bwd_resident_kernel<TG, TO, G, V, BLOCK, FAST, MASKED>),
                             dim3((unsigned)c.plan.grid), dim3(BLOCK), 0, c.stream,
                             (const TG*)c.a.grad, (const TG*)c.a.y, (TO*)c.a.gi,
                             MaskRef{c.a.mask, c.a.mask_div, c.a.mask_mod, c.a.mask_stride}, c.a.M, c.a.N,
                             c.a.flags);
          return true;
        }
      }
      return false;
    }
  };
};

template <class TG, class TO, bool MASKED>
int launch_softmax_bwd_m(const Plan& plan, const SoftmaxBwdArgs& a, hipStream_t stream) {
  if (plan.resident) {
    SoftmaxBwdCtx<TG, TO> ctx{plan, a, stream};
    const bool launched =
        plan.fast ? launch_variant<SoftmaxBwdLauncher<TG, TO, true, MASKED>::template At>(ctx)
                  : launch_variant<SoftmaxBwdLauncher<TG, TO, false, MASKED>::template At>(ctx);
    if (!launched) return (int)hipErrorInvalidConfiguration;
  } else {
    hipLaunchKernelGGL((softmax_bwd_stream_kernel<TG, TO, kStreamBlock, MASKED>),
                       dim3((unsigned)plan.grid), dim3(kStreamBlock), 0, stream,
                       (const TG*)a.grad, (const TG*)a.y, (TO*)a.gi,
                       MaskRef{a.mask, a.mask_div, a.mask_mod, a.mask_stride}, a.M, a.N, a.flags);
  }
  return (int)hipGetLastError();
}

template <class TG, class TO>
int launch_softmax_bwd(const Plan& plan, const SoftmaxBwdArgs& a, hipStream_t stream) {
  return a.mask ? launch_softmax_bwd_m<TG, TO, true>(plan, a, stream)
                : launch_softmax_bwd_m<TG, TO, false>(plan, a, stream);
}

}  // namespace rownorm
