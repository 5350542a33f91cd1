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
                    block_built(OC_SOFTMAX_FWD, G, BLOCK) &&
                    (!MASKED || masked_softmax_built(sizeof(TI), G, V))) {
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

template <class T, int LDSB>
bool launch_softmax_fwd_flat_l(FlatLayout f, int cr, const SoftmaxFwdArgs& a, hipStream_t stream) {
  const int64_t grid = (a.M + cr - 1) / cr;
  if (grid > 0x7fffffff) return false;
#define ROWNORM_FLAT_FWD(GL, VP)                                                                \
  case GL * 8 + VP:                                                                             \
    if constexpr (LDSB <= kFlatLdsBytes || (GL == 64 && VP >= 3)) {                             \
      hipLaunchKernelGGL((softmax_fwd_flat_kernel<T, GL, VP, kFlatBlock, LDSB>),                 \
                         dim3((unsigned)grid), dim3(kFlatBlock), 0, stream, (const T*)a.x,       \
                         (T*)a.y, a.M, a.N, cr, a.flags);                                       \
      return true;                                                                              \
    }                                                                                           \
    return false;
  switch (f.g * 8 + f.vp) { ROWNORM_FLAT_ALL(ROWNORM_FLAT_FWD) }
#undef ROWNORM_FLAT_FWD
  return false;
}

template <class T>
bool launch_softmax_fwd_flat(FlatLayout f, const SoftmaxFwdArgs& a, hipStream_t stream) {
  // 16 KB of LDS a workgroup; rows beyond 1024 16-bit elements (64 lanes, 3 or 4 packs) need 32 KB
  int cr = flat_chunk_rows<T>(a.N, f.g, kFlatLdsBytes);
  if (cr >= 8) return launch_softmax_fwd_flat_l<T, kFlatLdsBytes>(f, cr, a, stream);
  cr = flat_chunk_rows<T>(a.N, f.g, 2 * kFlatLdsBytes);
  if (cr >= 8) return launch_softmax_fwd_flat_l<T, 2 * kFlatLdsBytes>(f, cr, a, stream);
  return false;
}

template <class T, int LDSB>
bool launch_softmax_bwd_flat_l(FlatLayout f, int cr, const SoftmaxBwdArgs& a, hipStream_t stream) {
  const int64_t grid = (a.M + cr - 1) / cr;
  if (grid > 0x7fffffff) return false;
#define ROWNORM_FLAT_BWD(GL, VP)                                                                \
  case GL * 8 + VP:                                                                             \
    if constexpr ((LDSB == kFlatLdsBytes) || (LDSB < kFlatLdsBytes && GL <= 16) ||              \
                  (LDSB > kFlatLdsBytes && GL == 64 && VP >= 3)) {                              \
      hipLaunchKernelGGL((softmax_bwd_flat_kernel<T, GL, VP, kFlatBlock, LDSB>),                 \
                         dim3((unsigned)grid), dim3(kFlatBlock), 0, stream, (const T*)a.grad,    \
                         (const T*)a.y, (T*)a.gi, a.M, a.N, cr, a.flags);                       \
      return true;                                                                              \
    }                                                                                           \
    return false;
  switch (f.g * 8 + f.vp) { ROWNORM_FLAT_ALL(ROWNORM_FLAT_BWD) }
#undef ROWNORM_FLAT_BWD
  return false;
}

template <class T>
bool launch_softmax_bwd_flat(FlatLayout f, const SoftmaxBwdArgs& a, hipStream_t stream) {
  // per tensor: 8 KB where that still holds a full pass of the lane groups' rows (short
  // rows: more workgroups a compute unit), else 16 KB, else 32 KB (rows beyond 1024
  // 16-bit elements)
  const int rpb = kFlatBlock / f.g < 8 ? 8 : kFlatBlock / f.g;
  if (f.g <= 16) {
    const int half = flat_chunk_rows<T>(a.N, f.g, kFlatLdsBytes / 2);
    if (half >= rpb) return launch_softmax_bwd_flat_l<T, kFlatLdsBytes / 2>(f, half, a, stream);
  }
  int cr = flat_chunk_rows<T>(a.N, f.g, kFlatLdsBytes);
  if (cr >= 8) return launch_softmax_bwd_flat_l<T, kFlatLdsBytes>(f, cr, a, stream);
  cr = flat_chunk_rows<T>(a.N, f.g, 2 * kFlatLdsBytes);
  if (cr >= 8) return launch_softmax_bwd_flat_l<T, 2 * kFlatLdsBytes>(f, cr, a, stream);
  return false;
}

template <class TI, class TO, bool MASKED>
int launch_softmax_fwd_m(const Plan& plan, const SoftmaxFwdArgs& a, hipStream_t stream) {
  if constexpr (!MASKED && std::is_same<TI, TO>::value) {
    const FlatLayout f = flat_layout<TI>(plan, a.M, a.N, a.x, a.y, nullptr);
    if (f.g && launch_softmax_fwd_flat<TI>(f, a, stream)) return (int)hipGetLastError();
  }
  if constexpr (!MASKED) {
    if (plan.team > 0 && a.team_slot != nullptr) {
      // few very long rows: each in the registers of a team of workgroups
      TeamSlot* slot = (TeamSlot*)a.team_slot;
      auto go = [&](auto v) {
        constexpr int V = decltype(v)::value;
        hipLaunchKernelGGL((softmax_fwd_team_kernel<TI, TO, V>), dim3((unsigned)plan.team_grid),
                           dim3(kTeamBlock), 0, stream, (const TI*)a.x, (TO*)a.y, a.M, a.N, a.flags,
                           plan.team, plan.team_chunk_packs, slot, a.team_id, a.team_wait_ticks);
      };
      static_assert(kTeamMaxV == 16, "one case per pack count below");
      switch (plan.team_v) {
#define ROWNORM_TEAM_CASE(v) case v: go(std::integral_constant<int, v>{}); break;
        ROWNORM_TEAM_CASE(1) ROWNORM_TEAM_CASE(2) ROWNORM_TEAM_CASE(3) ROWNORM_TEAM_CASE(4)
        ROWNORM_TEAM_CASE(5) ROWNORM_TEAM_CASE(6) ROWNORM_TEAM_CASE(7) ROWNORM_TEAM_CASE(8)
        ROWNORM_TEAM_CASE(9) ROWNORM_TEAM_CASE(10) ROWNORM_TEAM_CASE(11) ROWNORM_TEAM_CASE(12)
        ROWNORM_TEAM_CASE(13) ROWNORM_TEAM_CASE(14) ROWNORM_TEAM_CASE(15) ROWNORM_TEAM_CASE(16)
#undef ROWNORM_TEAM_CASE
        default: return (int)hipErrorInvalidConfiguration;
      }
      return (int)hipGetLastError();
    }
  }
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
                    block_built(OC_SOFTMAX_BWD, G, BLOCK) &&
                    (!MASKED || masked_softmax_built(sizeof(TG), G, V))) {
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

// log_softmax backward of rows too long for both tensors in registers but not for
// grad alone: whole packs, 9 to 20 a lane on 1024 lanes (up to 8 both tensors fit:
// softmax_bwd_resident_kernel).  False: not this case.
template <class TG, class TO, int V>
inline void launch_grad_resident_v(const Plan& plan, const SoftmaxBwdArgs& a, hipStream_t stream) {
  hipLaunchKernelGGL((log_softmax_bwd_grad_resident_kernel<TG, TO, V, kStreamBlock>),
                     dim3((unsigned)plan.grid), dim3(kStreamBlock), 0, stream, (const TG*)a.grad,
                     (const TG*)a.y, (TO*)a.gi, a.M, a.N);
}

template <class TG, class TO>
inline bool launch_log_softmax_bwd_grad_resident(const Plan& plan, const SoftmaxBwdArgs& a,
                                                 hipStream_t stream) {
  constexpr int E = elems_per_pack<TG>::value;
  if (!plan.grad_resident || !(a.flags & kSoftmaxLog) || a.N % E != 0) return false;
  const int64_t packs = a.N / E;
  switch ((int)((packs + kStreamBlock - 1) / kStreamBlock)) {
    case 9: launch_grad_resident_v<TG, TO, 9>(plan, a, stream); return true;
    case 10: launch_grad_resident_v<TG, TO, 10>(plan, a, stream); return true;
    case 11: launch_grad_resident_v<TG, TO, 11>(plan, a, stream); return true;
    case 12: launch_grad_resident_v<TG, TO, 12>(plan, a, stream); return true;
    case 13: launch_grad_resident_v<TG, TO, 13>(plan, a, stream); return true;
    case 14: launch_grad_resident_v<TG, TO, 14>(plan, a, stream); return true;
    case 15: launch_grad_resident_v<TG, TO, 15>(plan, a, stream); return true;
    case 16: launch_grad_resident_v<TG, TO, 16>(plan, a, stream); return true;
    case 17: launch_grad_resident_v<TG, TO, 17>(plan, a, stream); return true;
    case 18: launch_grad_resident_v<TG, TO, 18>(plan, a, stream); return true;
    case 19: launch_grad_resident_v<TG, TO, 19>(plan, a, stream); return true;
    case 20: launch_grad_resident_v<TG, TO, 20>(plan, a, stream); return true;
  }
  return false;
}

template <class TG, class TO, bool MASKED>
int launch_softmax_bwd_m(const Plan& plan, const SoftmaxBwdArgs& a, hipStream_t stream) {
  if constexpr (!MASKED && std::is_same<TG, TO>::value) {
    const FlatLayout f = flat_layout<TG>(plan, a.M, a.N, a.grad, a.y, a.gi);
    if (f.g && launch_softmax_bwd_flat<TG>(f, a, stream)) return (int)hipGetLastError();
  }
  if constexpr (!MASKED) {
    if (plan.team > 0 && a.team_slot != nullptr) {
      // few very long rows: each in the registers of a team of workgroups
      TeamSlot* slot = (TeamSlot*)a.team_slot;
      auto go = [&](auto v) {
        constexpr int V = decltype(v)::value;
        hipLaunchKernelGGL((softmax_bwd_team_kernel<TG, TO, V>), dim3((unsigned)plan.team_grid),
                           dim3(kTeamBlock), 0, stream, (const TG*)a.grad, (const TG*)a.y,
                           (TO*)a.gi, a.M, a.N, a.flags, plan.team, plan.team_chunk_packs, slot,
                           a.team_id, a.team_wait_ticks);
      };
      static_assert(kSoftmaxBwdTeamMaxV == 8, "one case per pack count below");
      switch (plan.team_v) {
#define ROWNORM_TEAM_CASE(v) case v: go(std::integral_constant<int, v>{}); break;
        ROWNORM_TEAM_CASE(1) ROWNORM_TEAM_CASE(2) ROWNORM_TEAM_CASE(3) ROWNORM_TEAM_CASE(4)
        ROWNORM_TEAM_CASE(5) ROWNORM_TEAM_CASE(6) ROWNORM_TEAM_CASE(7) ROWNORM_TEAM_CASE(8)
#undef ROWNORM_TEAM_CASE
        default: return (int)hipErrorInvalidConfiguration;
      }
      return (int)hipGetLastError();
    }
  }
  if (plan.resident) {
    SoftmaxBwdCtx<TG, TO> ctx{plan, a, stream};
    const bool launched =
        plan.fast ? launch_variant<SoftmaxBwdLauncher<TG, TO, true, MASKED>::template At>(ctx)
                  : launch_variant<SoftmaxBwdLauncher<TG, TO, false, MASKED>::template At>(ctx);
    if (!launched) return (int)hipErrorInvalidConfiguration;
  } else if (!MASKED && launch_log_softmax_bwd_grad_resident<TG, TO>(plan, a, stream)) {
    // (log_softmax rows of up to 16 packs a lane: grad resident, y streamed)
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
