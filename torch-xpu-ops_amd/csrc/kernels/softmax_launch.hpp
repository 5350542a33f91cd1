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

// Short ragged rows through LDS (softmax_fwd_flat_kernel / softmax_bwd_flat_kernel).
constexpr int kFlatWholePackRowsMaxPacks = 12;
struct FlatLayout {
  int g = 0;   // lanes per row (0: the call does not qualify)
  int vp = 0;  // packs per lane
};

// The (lanes 4..64, packs per lane 1..4) with the fewest idle pack slots; among
// equals the one nearest two packs a lane, the layout the resident kernels prefer.
// Measured against "two packs a lane on the fewest lanes that hold the row",
// interleaved, bf16 forward / backward in us: rows of 13: 19.5 / 18.5 -> 10.6 / 8.6,
// 21: 30.0 / 25.9 -> 14.1 / 16.1, 45: 20.3 / 22.8 -> 16.5 / 20.6, 577 (73 packs: 32 x 3
// instead of 64 x 2): 72.1 / 96.5 -> 67.8 / 96.3, 750: 54.0 / 76.2 -> 51.2 / 75.1; 93
// and 129 lose 5-10 % in the backward (13.1 -> 14.6, 33.1 -> 34.8).
template <class T>
inline FlatLayout flat_layout(const Plan& plan, int64_t M, int N, const void* p0, const void* p1,
                              const void* p2) {
  constexpr int E = elems_per_pack<T>::value;
  FlatLayout f;
  if (plan.forced || M < 1 || N > 64 * kFlatMaxPacks * E) return f;
  if ((((uintptr_t)p0) | ((uintptr_t)p1) | ((uintptr_t)p2)) & 15) return f;
  const int packs = (N + E - 1) / E;
  // rows of whole packs qualify only when they are very short (see below)
  if (plan.fast && (packs > kFlatWholePackRowsMaxPacks || !plan.resident)) return f;
  int best_slots = 0, best_rank = 0;
  for (int g = 4; g <= 64; g <<= 1) {
    const int vp = (packs + g - 1) / g;
    if (vp > kFlatMaxPacks) continue;
    const int slots = g * vp;
    const int rank = vp == 2 ? 0 : (vp == 3 ? 1 : (vp == 1 ? 2 : 3));
    if (f.g == 0 || slots < best_slots || (slots == best_slots && rank < best_rank)) {
      f.g = g;
      f.vp = vp;
      best_slots = slots;
      best_rank = rank;
    }
  }
  // Rows of whole packs: only up to 12 packs and where the resident layout leaves a
  // quarter of its pack slots idle, e.g. 9 or 10 packs on 8 lanes x 2 (bf16 rows of 72:
  // 36.6 / 52.5 -> 31.2 / 44.3 us, of 80: 40.9 / 57.6 -> 33.2 / 48.2 us, of 24: 32.1 / 29.4
  // -> 18.1 / 25.1 us); from 17 packs on it measured the same or slower (520: +2 %, 1032:
  // the backward +30 %).
  if (plan.fast && best_slots * 4 > plan.G * plan.V * 3) f = FlatLayout{};
  return f;
}

// One case per (lanes, packs per lane) of a launch switch keyed by lanes * 8 + packs.
#define ROWNORM_FLAT_CASES(CASE, GL) CASE(GL, 1) CASE(GL, 2) CASE(GL, 3) CASE(GL, 4)
#define ROWNORM_FLAT_ALL(CASE)                                                       \
  ROWNORM_FLAT_CASES(CASE, 4) ROWNORM_FLAT_CASES(CASE, 8) ROWNORM_FLAT_CASES(CASE, 16) \
  ROWNORM_FLAT_CASES(CASE, 32) ROWNORM_FLAT_CASES(CASE, 64)

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
