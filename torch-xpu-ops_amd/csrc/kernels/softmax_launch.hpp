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

template <class TI, class TO, bool FAST>
struct SoftmaxFwdLauncher {
  template <int G, int V, int BLOCK>
  struct At {
    static bool run(const SoftmaxFwdCtx<TI, TO>& c) {
      if constexpr (variant_built(OC_SOFTMAX_FWD, sizeof(TI), G, V, FAST) &&
                    block_built(OC_SOFTMAX_FWD, G, BLOCK)) {
        if (c.plan.G == G && c.plan.V == V && c.plan.block == BLOCK) {
          hipLaunchKernelGGL((softmax_fwd_resident_kernel<TI, TO, G, V, BLOCK, FAST>),
                             dim3((unsigned)c.plan.grid), dim3(BLOCK), 0, c.stream,
                             (const TI*)c.a.x, (TO*)c.a.y, c.a.M, c.a.N, c.a.is_log);
          return true;
        }
      }
      return false;
    }
  };
};

template <class TI, class TO>
int launch_softmax_fwd(const Plan& plan, const SoftmaxFwdArgs& a, hipStream_t stream) {
  if (plan.resident) {
    SoftmaxFwdCtx<TI, TO> ctx{plan, a, stream};
    const bool launched =
        plan.fast ? launch_variant<SoftmaxFwdLauncher<TI, TO, true>::template At>(ctx)
                  : launch_variant<SoftmaxFwdLauncher<TI, TO, false>::template At>(ctx);
    if (!launched) return (int)hipErrorInvalidConfiguration;
  } else {
    hipLaunchKernelGGL((softmax_fwd_stream_kernel<TI, TO, kStreamBlock>),
                       dim3((unsigned)plan.grid), dim3(kStreamBlock), 0, stream, (const TI*)a.x,
                       (TO*)a.y, a.M, a.N, a.is_log);
  }
  return (int)hipGetLastError();
}

template <class TG, class TO>
struct SoftmaxBwdCtx {
  const Plan& plan;
  const SoftmaxBwdArgs& a;
  hipStream_t stream;
};

template <class TG, class TO, bool FAST>
struct SoftmaxBwdLauncher {
  template <int G, int V, int BLOCK>
  struct At {
    static bool run(const SoftmaxBwdCtx<TG, TO>& c) {
      if constexpr (variant_built(OC_SOFTMAX_BWD, sizeof(TG), G, V, FAST) &&
                    block_built(OC_SOFTMAX_BWD, G, BLOCK)) {
        if (c.plan.G == G && c.plan.V == V && c.plan.block == BLOCK) {
          hipLaunchKernelGGL((softmax_bwd_resident_kernel<TG, TO, G, V, BLOCK, FAST>),
                             dim3((unsigned)c.plan.grid), dim3(BLOCK), 0, c.stream,
                             (const TG*)c.a.grad, (const TG*)c.a.y, (TO*)c.a.gi, c.a.M, c.a.N,
                             c.a.is_log);
          return true;
        }
      }
      return false;
    }
  };
};

template <class TG, class TO>
int launch_softmax_bwd(const Plan& plan, const SoftmaxBwdArgs& a, hipStream_t stream) {
  if (plan.resident) {
    SoftmaxBwdCtx<TG, TO> ctx{plan, a, stream};
    const bool launched =
        plan.fast ? launch_variant<SoftmaxBwdLauncher<TG, TO, true>::template At>(ctx)
                  : launch_variant<SoftmaxBwdLauncher<TG, TO, false>::template At>(ctx);
    if (!launched) return (int)hipErrorInvalidConfiguration;
  } else {
    hipLaunchKernelGGL((softmax_bwd_stream_kernel<TG, TO, kStreamBlock>),
                       dim3((unsigned)plan.grid), dim3(kStreamBlock), 0, stream,
                       (const TG*)a.grad, (const TG*)a.y, (TO*)a.gi, a.M, a.N, a.is_log);
  }
  return (int)hipGetLastError();
}

}  // namespace rownorm
