// Host dispatch of the GroupNorm kernels: plan -> template instance.
#pragma once
#include "groupnorm_kernels.hpp"
#include "launch.hpp"
#include "norm_kernels.hpp"  // colsum_finalize_kernel

namespace rownorm {

// E: elements per pack of the row dtype.
inline GroupShape group_shape(int L, int HxW, int D, int groups, int E) {
  GroupShape s{L, HxW, D, groups, 0, 0u, 0u};
  const int mode = gn_mode(L, HxW, D, E);
  if (mode == kGnUniform) {
    const uint64_t per_channel = (uint64_t)(HxW / E);
    s.packs = L / E;
    s.pack_magic = (unsigned)((((uint64_t)1 << 31) + per_channel - 1) / per_channel);
  } else if (mode == kGnStraddle) {
    s.elem_magic = (unsigned)((((uint64_t)1 << 32) + (uint64_t)HxW - 1) / (uint64_t)HxW);
  }
  return s;
}

template <class T, class WT>
struct GroupNormFwdCtx {
  const Plan& plan;
  const GroupNormFwdArgs& a;
  hipStream_t stream;
};

template <class T, class WT, int MODE>
struct GroupNormFwdLauncher {
  template <int G, int V, int BLOCK>
  struct At {
    static bool run(const GroupNormFwdCtx<T, WT>& c) {
      if constexpr (variant_built(OC_GROUP_FWD, sizeof(T), G, V, MODE != kGnGeneral) &&
                    block_built(OC_GROUP_FWD, G, BLOCK)) {
        if (c.plan.G == G && c.plan.V == V && c.plan.block == BLOCK) {
          hipLaunchKernelGGL((gn_fwd_resident_kernel<T, WT, G, V, BLOCK, MODE>),
                             dim3((unsigned)c.plan.grid), dim3(BLOCK), 0, c.stream,
                             (const T*)c.a.x, (const WT*)c.a.gamma, (const WT*)c.a.beta,
                             (T*)c.a.y, (WT*)c.a.mean, (WT*)c.a.rstd, c.a.rows,
                             group_shape(c.a.L, c.a.HxW, c.a.D, c.a.groups, elems_per_pack<T>::value), c.a.eps);
          return true;
        }
      }
      return false;
    }
  };
};

// The exact layouts (kGroupExact): entry I of the table, if the plan names it.
template <class T, class WT, int I>
inline bool launch_group_fwd_exact_at(const Plan& plan, const GroupNormFwdArgs& a,
                                      hipStream_t stream) {
  constexpr GroupExactLayout l = kGroupExact[I];
  if constexpr (sizeof(T) == 2 && l.bpc_fwd > 0) {
    if (plan.G == l.G && plan.V == l.V) {
      hipLaunchKernelGGL((gn_fwd_exact_kernel<T, WT, l.G, l.V>), dim3((unsigned)plan.grid),
                         dim3(l.G), 0, stream, (const T*)a.x, (const WT*)a.gamma,
                         (const WT*)a.beta, (T*)a.y, (WT*)a.mean, (WT*)a.rstd, a.rows,
                         group_shape(a.L, a.HxW, a.D, a.groups, elems_per_pack<T>::value), a.eps);
      return true;
    }
  }
  return false;
}
template <class T, class WT, int... Is>
inline bool launch_group_fwd_exact(const Plan& plan, const GroupNormFwdArgs& a, hipStream_t stream,
                                   ilist<Is...>) {
  return (launch_group_fwd_exact_at<T, WT, Is>(plan, a, stream) || ...);
}

template <class T, class WT>
int launch_group_norm_fwd(const Plan& plan, const GroupNormFwdArgs& a, hipStream_t stream) {
  if (plan.resident && plan.exact_depth > 0) {
    static_assert(kGroupExactCount == 5, "one index per table entry below");
    if (!launch_group_fwd_exact<T, WT>(plan, a, stream, ilist<0, 1, 2, 3, 4>{}))
      return (int)hipErrorInvalidConfiguration;
  } else if (plan.resident) {
    GroupNormFwdCtx<T, WT> ctx{plan, a, stream};
    const int mode = plan.fast ? gn_mode(a.L, a.HxW, a.D, elems_per_pack<T>::value) : kGnGeneral;
    const bool launched =
        mode == kGnUniform    ? launch_variant<GroupNormFwdLauncher<T, WT, kGnUniform>::template At>(ctx)
        : mode == kGnStraddle ? launch_variant<GroupNormFwdLauncher<T, WT, kGnStraddle>::template At>(ctx)
                              : launch_variant<GroupNormFwdLauncher<T, WT, kGnGeneral>::template At>(ctx);
    if (!launched) return (int)hipErrorInvalidConfiguration;
  } else if (plan.team > 0 && a.team_slot != nullptr &&
             a.HxW % elems_per_pack<T>::value == 0) {
    // slabs beyond one workgroup's registers whose channels are whole packs: one pass,
    // a slab in the registers of a team of workgroups (norm_fwd_team_kernel, GROUP)
    TeamGroupShape gs;
    gs.groups = a.groups;
    gs.channels = a.D;
    gs.packs_per_channel = a.HxW / elems_per_pack<T>::value;
    auto go = [&](auto v) {
      constexpr int V = decltype(v)::value;
      hipLaunchKernelGGL((norm_fwd_team_kernel<T, WT, V, false, true, WT>),
                         dim3((unsigned)plan.team_grid), dim3(kTeamBlock), 0, stream,
                         (const T*)a.x, (const WT*)a.gamma, (const WT*)a.beta, (T*)a.y,
                         (WT*)a.mean, (WT*)a.rstd, a.rows, a.L, a.eps, plan.team,
                         plan.team_chunk_packs, (TeamSlot*)a.team_slot, a.team_id,
                         a.team_wait_ticks, gs);
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
  } else {
    hipLaunchKernelGGL((gn_fwd_stream_kernel<T, WT, kStreamBlock>), dim3((unsigned)plan.grid),
                       dim3(kStreamBlock), 0, stream, (const T*)a.x, (const WT*)a.gamma,
                       (const WT*)a.beta, (T*)a.y, (WT*)a.mean, (WT*)a.rstd, a.rows,
                       group_shape(a.L, a.HxW, a.D, a.groups, elems_per_pack<T>::value), a.eps);
  }
  return (int)hipGetLastError();
}

template <class T, class WT>
struct GroupNormBwdCtx {
  const Plan& plan;
  const GroupNormBwdArgs& a;
  int tpc_log2;
  hipStream_t stream;
};

template <class T, class WT, int MODE>
struct GroupNormBwdLauncher {
  template <int G, int V, int BLOCK>
  struct At {
    static bool run(const GroupNormBwdCtx<T, WT>& c) {
      if constexpr (variant_built(OC_GROUP_BWD, sizeof(T), G, V, MODE != kGnGeneral) &&
                    block_built(OC_GROUP_BWD, G, BLOCK)) {
        if (c.plan.G == G && c.plan.V == V && c.plan.block == BLOCK) {
          hipLaunchKernelGGL((gn_bwd_resident_kernel<T, WT, G, V, BLOCK, MODE>),
                             dim3((unsigned)c.plan.grid), dim3(BLOCK), 0, c.stream,
                             (const T*)c.a.dy, (const T*)c.a.x, (const WT*)c.a.mean,
                             (const WT*)c.a.rstd, (const WT*)c.a.gamma, (T*)c.a.dx, c.a.part_dg,
                             c.a.part_db, c.a.rows,
                             group_shape(c.a.L, c.a.HxW, c.a.D, c.a.groups, elems_per_pack<T>::value), c.tpc_log2);
          return true;
        }
      }
      return false;
    }
  };
};

// Lanes that share one channel in the fused channel sums: as many as the row
// group has to spare for its D channels, at most a wavefront, at most the packs
// of a channel.
inline int gn_tpc_log2(int G, int D, int packs_per_channel) {
  int tpc = G / pow2_ceil(D);
  if (tpc > 64) tpc = 64;
  while (tpc > 1 && tpc > packs_per_channel) tpc >>= 1;
  if (tpc < 1) tpc = 1;
  return log2_of_pow2(tpc);
}

template <class T, class WT, int I>
inline bool launch_group_bwd_exact_at(const Plan& plan, const GroupNormBwdArgs& a,
                                      hipStream_t stream) {
  constexpr GroupExactLayout l = kGroupExact[I];
  if constexpr (sizeof(T) == 2 && l.bpc_bwd > 0) {
    if (plan.G == l.G && plan.V == l.V) {
      const GroupShape shape = group_shape(a.L, a.HxW, a.D, a.groups, elems_per_pack<T>::value);
      if (a.part_dg != nullptr)
        hipLaunchKernelGGL((gn_bwd_exact_kernel<T, WT, l.G, l.V, true>), dim3((unsigned)plan.grid),
                           dim3(l.G), 0, stream, (const T*)a.dy, (const T*)a.x, (const WT*)a.mean,
                           (const WT*)a.rstd, (const WT*)a.gamma, (T*)a.dx, a.part_dg, a.part_db,
                           a.rows, shape);
      else
        hipLaunchKernelGGL((gn_bwd_exact_kernel<T, WT, l.G, l.V, false>), dim3((unsigned)plan.grid),
                           dim3(l.G), 0, stream, (const T*)a.dy, (const T*)a.x, (const WT*)a.mean,
                           (const WT*)a.rstd, (const WT*)a.gamma, (T*)a.dx, a.part_dg, a.part_db,
                           a.rows, shape);
      return true;
    }
  }
  return false;
}
template <class T, class WT, int... Is>
inline bool launch_group_bwd_exact(const Plan& plan, const GroupNormBwdArgs& a, hipStream_t stream,
                                   ilist<Is...>) {
  return (launch_group_bwd_exact_at<T, WT, Is>(plan, a, stream) || ...);
}

// Partial rows (one a sample) the second stage of the backward folds in place at a time, where
// there are very many samples.
constexpr int kGnFoldRows = 512;

template <class T, class WT>
int launch_group_norm_bwd(const Plan& plan, const GroupNormBwdArgs& a, hipStream_t stream) {
  constexpr int E = elems_per_pack<T>::value;
  const bool want_cols = a.dgamma != nullptr || a.dbeta != nullptr;
  const bool fused_cols = plan.resident && plan.fast;  // channel sums come out of the dX kernel
  // rows too long for the registers get dX from the channel sums, wanted or not
  const bool need_sums = want_cols || (!plan.resident && a.dx != nullptr);
  const GroupShape shape = group_shape(a.L, a.HxW, a.D, a.groups, elems_per_pack<T>::value);
  const int64_t N = a.rows / a.groups;
  const int C = a.groups * a.D;
  int err = 0;
  const bool teams = !plan.resident && a.team > 0 && a.team_slot != nullptr && a.dx != nullptr;
  if (teams) {
    // slabs beyond the registers, dY and X read once: teams of workgroups
    GroupNormBwdArgs k = a;
    if (!want_cols) k.part_dg = k.part_db = nullptr;
    auto go = [&](auto v) {
      constexpr int V = decltype(v)::value;
      hipLaunchKernelGGL((gn_bwd_team_kernel<T, WT, V>), dim3((unsigned)a.team_grid),
                         dim3(kTeamBlock), 0, stream, (const T*)a.dy, (const T*)a.x,
                         (const WT*)a.mean, (const WT*)a.rstd, (const WT*)a.gamma, (T*)a.dx,
                         k.part_dg, k.part_db, a.rows, shape, a.team, a.team_wpc,
                         (TeamSlot*)a.team_slot, a.team_id, a.team_wait_ticks);
    };
    switch (a.team_v) {
      case 4: go(std::integral_constant<int, 4>{}); break;
      case 8: go(std::integral_constant<int, 8>{}); break;
      default: return (int)hipErrorInvalidConfiguration;
    }
  } else if (need_sums && !fused_cols) {
    const int packs = (a.HxW + E - 1) / E;
    const int64_t nc_rows = N * C;
    auto sums = [&](auto cb) {
      constexpr int CB = decltype(cb)::value;
      // long channel rows take a whole workgroup each
      const int lanes = packs >= 8 * CB ? CB : (packs >= 64 ? 64 : pow2_ceil(packs));
      const int rpb = CB / lanes;
      int64_t grid = (nc_rows + rpb - 1) / rpb;
      if (grid > (1 << 22)) grid = 1 << 22;
      hipLaunchKernelGGL((gn_channel_sums_kernel<T, WT, CB>), dim3((unsigned)grid), dim3(CB), 0,
                         stream, (const T*)a.dy, (const T*)a.x, (const WT*)a.mean,
                         (const WT*)a.rstd, a.part_dg, a.part_db, nc_rows, shape,
                         log2_of_pow2(lanes));
    };
    // (channel rows of 8192 packs and more -- 256 x 256 maps in 16 bits -- on 1024 threads:
    // there are few of them, and each lane keeps four pack pairs in flight)
    if (packs >= 8 * 1024)
      sums(std::integral_constant<int, 1024>{});
    else
      sums(std::integral_constant<int, 256>{});
    err = (int)hipGetLastError();
    if (err != 0) return err;
  }
  if (teams) {
    // (launched above)
  } else if (plan.resident && plan.exact_depth > 0) {
    GroupNormBwdArgs k = a;
    if (!want_cols) k.part_dg = k.part_db = nullptr;
    if (a.dx == nullptr || !launch_group_bwd_exact<T, WT>(plan, k, stream, ilist<0, 1, 2, 3, 4>{}))
      return (int)hipErrorInvalidConfiguration;
  } else if (plan.resident) {
    if (a.dx != nullptr || (want_cols && fused_cols)) {
      GroupNormBwdArgs k = a;
      if (!want_cols || !fused_cols) k.part_dg = k.part_db = nullptr;
      GroupNormBwdCtx<T, WT> ctx{plan, k, 0, stream};
      if (plan.fast) ctx.tpc_log2 = gn_tpc_log2(plan.G, a.D, a.HxW / E);
      const int mode = plan.fast ? gn_mode(a.L, a.HxW, a.D, E) : kGnGeneral;
      const bool launched =
          mode == kGnUniform    ? launch_variant<GroupNormBwdLauncher<T, WT, kGnUniform>::template At>(ctx)
          : mode == kGnStraddle ? launch_variant<GroupNormBwdLauncher<T, WT, kGnStraddle>::template At>(ctx)
                                : launch_variant<GroupNormBwdLauncher<T, WT, kGnGeneral>::template At>(ctx);
      if (!launched) return (int)hipErrorInvalidConfiguration;
    }
  } else if (a.dx != nullptr) {
    constexpr int DB = 256;
    const int64_t chunk_elems = (int64_t)DB * kGnChunkPacks * E;
    const int chunks = (int)((a.L + chunk_elems - 1) / chunk_elems);
    int64_t grid = a.rows * chunks;
    if (grid > (1 << 24)) grid = 1 << 24;
    hipLaunchKernelGGL((gn_bwd_dx_from_sums_kernel<T, WT, DB>), dim3((unsigned)grid), dim3(DB), 0,
                       stream, (const T*)a.dy, (const T*)a.x, (const WT*)a.mean,
                       (const WT*)a.rstd, (const WT*)a.gamma, (const float*)a.part_dg,
                       (const float*)a.part_db, (T*)a.dx, a.rows, shape, chunks);
  }
  err = (int)hipGetLastError();
  if (err != 0 || !want_cols) return err;
  const unsigned gx = (unsigned)((C + kFinalizeCols - 1) / kFinalizeCols);
  // one partial row a sample: with very many samples under few channels the rows are first
  // folded in place, kGnFoldRows at a time, by as many workgroups as that gives (bf16
  // [1048576, 32] in 8 groups: the second stage alone took 4 ms on its one workgroup)
  if (N >= 16 * kGnFoldRows && N <= 65535 * (int64_t)kGnFoldRows && gx <= 32) {
    const unsigned folds = (unsigned)((N + kGnFoldRows - 1) / kGnFoldRows);
    hipLaunchKernelGGL((colsum_finalize_kernel<float, true>), dim3(gx, 2, folds), dim3(1024), 0,
                       stream, (const float*)a.part_dg, (const float*)a.part_db, (float*)nullptr,
                       (float*)nullptr, (int)N, C, (int64_t)C, kGnFoldRows);
    hipLaunchKernelGGL((colsum_finalize_kernel<WT>), dim3(gx, 2), dim3(1024), 0, stream,
                       (const float*)a.part_dg, (const float*)a.part_db, (WT*)a.dgamma,
                       (WT*)a.dbeta, (int)folds, C, (int64_t)kGnFoldRows * C, 0);
    return (int)hipGetLastError();
  }
  hipLaunchKernelGGL((colsum_finalize_kernel<WT>), dim3(gx, 2), dim3(1024), 0, stream,
                     (const float*)a.part_dg, (const float*)a.part_db, (WT*)a.dgamma,
                     (WT*)a.dbeta, (int)N, C);
  return (int)hipGetLastError();
}

}  // namespace rownorm
