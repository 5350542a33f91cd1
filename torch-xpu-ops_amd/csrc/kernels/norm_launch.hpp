// Host dispatch of the LayerNorm / RMSNorm kernels: plan -> template instance.
#pragma once
#include "launch.hpp"
#include "norm_kernels.hpp"

namespace rownorm {

template <class T, class WT, bool RMS>
struct NormFwdCtx {
  const Plan& plan;
  const NormFwdArgs& a;
  hipStream_t stream;
};

template <class T, class WT, bool RMS, bool FAST, class TY, bool ADD>
struct NormFwdLauncher {
  template <int G, int V, int BLOCK>
  struct At {
    static bool run(const NormFwdCtx<T, WT, RMS>& c) {
      if constexpr (variant_built(OC_NORM_FWD, sizeof(T), G, V, FAST) &&
                    block_built(OC_NORM_FWD, G, BLOCK)) {
        if (c.plan.G == G && c.plan.V == V && c.plan.block == BLOCK) {
          hipLaunchKernelGGL(
              (norm_fwd_resident_kernel<T, WT, G, V, BLOCK, 1, RMS, FAST, TY, ADD>),
              dim3((unsigned)c.plan.grid), dim3(BLOCK), 0, c.stream, (const T*)c.a.x,
              (const T*)c.a.res, (const WT*)c.a.gamma, (const WT*)c.a.beta, (T*)c.a.h,
              (TY*)c.a.y, c.a.mean, c.a.rstd, c.a.M, c.a.N, c.a.eps);
          return true;
        }
      }
      return false;
    }
  };
};

// The split-row forward keeps a chunk's partial sums in the first bytes of the
// chunk's piece of Y and hands the statistics to its last launch through mean /
// rstd: it needs those outputs, and a Y that overlaps none of X, res and h.
template <class T, class TY, bool RMS>
inline bool norm_fwd_can_split(const Plan& plan, const NormFwdArgs& a) {
  if (plan.split <= 1 || a.M > 65535 || a.rstd == nullptr || (!RMS && a.mean == nullptr))
    return false;
  const int64_t elems = a.M * (int64_t)a.N;
  const int64_t ybytes = elems * (int64_t)sizeof(TY), xbytes = elems * (int64_t)sizeof(T);
  return regions_disjoint(a.y, ybytes, a.x, xbytes) && regions_disjoint(a.y, ybytes, a.res, xbytes) &&
         regions_disjoint(a.y, ybytes, a.h, xbytes);
}

// Whether norm_fwd_team_kernel serves the call: planned, its bookkeeping memory at
// hand (the caller of this function withholds it on a stream under capture), no
// residual add, Y in the row dtype.  (The caller also withholds the memory when Y
// overlaps X: a workgroup whose team does not come together reads the whole row.)
template <class T, class TY, bool ADD>
inline bool norm_fwd_team_serves(const Plan& plan, const NormFwdArgs& a) {
  return plan.team > 0 && a.team_slot != nullptr && !ADD && std::is_same<T, TY>::value &&
         a.res == nullptr;
}

// The exact two-pack forward layouts (kNormFwdExact): entry I of the table, if the plan names it.
template <class T, class WT, bool RMS, int I>
inline bool launch_norm_fwd_exact_at(const Plan& plan, const NormFwdArgs& a, hipStream_t stream) {
  constexpr NormFwdExactLayout l = kNormFwdExact[I];
  if constexpr (sizeof(T) == 2) {
    if (plan.G == l.G && plan.block == l.block) {
      hipLaunchKernelGGL((norm_fwd_exact_kernel<T, WT, l.G, l.block, RMS>),
                         dim3((unsigned)plan.grid), dim3(l.block), 0, stream, (const T*)a.x,
                         (const WT*)a.gamma, (const WT*)a.beta, (T*)a.y, a.mean, a.rstd, a.M, a.N,
                         a.eps);
      return true;
    }
  }
  return false;
}

// Short ragged rows through LDS (norm_fwd_flat_kernel): 16 KB a workgroup, 32 KB for rows
// beyond 1024 16-bit elements.
template <class T, class WT, bool RMS, int LDSB>
bool launch_norm_fwd_flat_l(FlatLayout f, int cr, const NormFwdArgs& a, hipStream_t stream) {
  const int64_t grid = (a.M + cr - 1) / cr;
  if (grid > 0x7fffffff) return false;
#define ROWNORM_FLAT_NORM_FWD(GL, VP)                                                           \
  case GL * 8 + VP:                                                                             \
    if constexpr (LDSB <= kFlatLdsBytes || (GL == 64 && VP >= 3)) {                             \
      hipLaunchKernelGGL((norm_fwd_flat_kernel<T, WT, GL, VP, kFlatBlock, LDSB, RMS>),           \
                         dim3((unsigned)grid), dim3(kFlatBlock), 0, stream, (const T*)a.x,       \
                         (const WT*)a.gamma, (const WT*)a.beta, (T*)a.y, a.mean, a.rstd, a.M,    \
                         a.N, cr, a.eps);                                                       \
      return true;                                                                              \
    }                                                                                           \
    return false;
  switch (f.g * 8 + f.vp) { ROWNORM_FLAT_ALL(ROWNORM_FLAT_NORM_FWD) }
#undef ROWNORM_FLAT_NORM_FWD
  return false;
}

template <class T, class WT, bool RMS>
bool launch_norm_fwd_flat(FlatLayout f, const NormFwdArgs& a, hipStream_t stream) {
  int cr = flat_chunk_rows<T>(a.N, f.g, kFlatLdsBytes);
  if (cr >= 8) return launch_norm_fwd_flat_l<T, WT, RMS, kFlatLdsBytes>(f, cr, a, stream);
  cr = flat_chunk_rows<T>(a.N, f.g, 2 * kFlatLdsBytes);
  if (cr >= 8) return launch_norm_fwd_flat_l<T, WT, RMS, 2 * kFlatLdsBytes>(f, cr, a, stream);
  return false;
}

template <class T, class WT, bool RMS, class TY, bool ADD>
int launch_norm_fwd(const Plan& plan, const NormFwdArgs& a, hipStream_t stream) {
  const T* res = ADD ? (const T*)a.res : nullptr;
  T* h = ADD ? (T*)a.h : nullptr;
  // short ragged rows (no residual add, no cast, 16-byte aligned X and Y): staged through LDS
  if constexpr (!ADD && std::is_same<T, TY>::value) {
    if (plan.resident && plan.exact_depth == 0 && !plan.window) {
      const FlatLayout f = flat_layout<T>(plan, a.M, a.N, a.x, a.y, nullptr);
      if (f.g != 0 && launch_norm_fwd_flat<T, WT, RMS>(f, a, stream))
        return (int)hipGetLastError();
    }
  }
  if (norm_fwd_team_serves<T, TY, ADD>(plan, a) && plan.team_r > 0) {
    // one pass with three rows in flight in the registers of a team of workgroups, weights held
    if constexpr (!ADD && std::is_same<T, TY>::value) {
      TeamSlot* slot = (TeamSlot*)a.team_slot;
      auto go = [&](auto r, auto v) {
        constexpr int R = decltype(r)::value, V = decltype(v)::value;
        hipLaunchKernelGGL((norm_fwd_rows_team_kernel<T, WT, RMS, R, V>),
                           dim3((unsigned)plan.team_grid), dim3(kTeamBlock), 0, stream,
                           (const T*)a.x, (const WT*)a.gamma, (const WT*)a.beta, (T*)a.y, a.mean,
                           a.rstd, a.M, a.N, a.eps, plan.team, slot, a.team_id, a.team_wait_ticks);
      };
      if (sizeof(WT) == sizeof(T) && plan.team_r == 1 && plan.team_v == kTeamFwdLongPacks) {
        if constexpr (sizeof(WT) == sizeof(T))
          go(std::integral_constant<int, 1>{}, std::integral_constant<int, kTeamFwdLongPacks>{});
      } else {
        return (int)hipErrorInvalidConfiguration;
      }
    }
  } else if (norm_fwd_team_serves<T, TY, ADD>(plan, a)) {
    // one pass with the row in the registers of a team of workgroups
    TeamSlot* slot = (TeamSlot*)a.team_slot;
    auto go = [&](auto v) {
      constexpr int V = decltype(v)::value;
      hipLaunchKernelGGL((norm_fwd_team_kernel<T, WT, V, RMS>), dim3((unsigned)plan.team_grid),
                         dim3(kTeamBlock), 0, stream, (const T*)a.x, (const WT*)a.gamma,
                         (const WT*)a.beta, (T*)a.y, a.mean, a.rstd, a.M, a.N, a.eps, plan.team,
                         plan.team_chunk_packs, slot, a.team_id, a.team_wait_ticks);
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
  } else if (plan.resident && plan.exact_depth > 0) {
    static_assert(kNormFwdExactCount == 2, "one call per table entry below");
    bool launched = false;
    if constexpr (!ADD && std::is_same<T, TY>::value)
      launched = launch_norm_fwd_exact_at<T, WT, RMS, 0>(plan, a, stream) ||
                 launch_norm_fwd_exact_at<T, WT, RMS, 1>(plan, a, stream);
    if (!launched) return (int)hipErrorInvalidConfiguration;
  } else if (plan.resident) {
    NormFwdCtx<T, WT, RMS> ctx{plan, a, stream};
    const bool launched =
        plan.fast
            ? launch_variant<NormFwdLauncher<T, WT, RMS, true, TY, ADD>::template At>(ctx)
            : launch_variant<NormFwdLauncher<T, WT, RMS, false, TY, ADD>::template At>(ctx);
    if (!launched) return (int)hipErrorInvalidConfiguration;
  } else if (norm_fwd_can_split<T, TY, RMS>(plan, a)) {
    const dim3 grid((unsigned)plan.split, (unsigned)a.M);
    hipLaunchKernelGGL((norm_fwd_split_sums_kernel<T, kStreamBlock, RMS, TY>), grid,
                       dim3(kStreamBlock), 0, stream, (const T*)a.x, res, (TY*)a.y, a.N,
                       plan.chunk_packs);
    hipLaunchKernelGGL((norm_fwd_split_stats_kernel<T, RMS, TY>), dim3((unsigned)a.M), dim3(64), 0,
                       stream, (const T*)a.x, res, (TY*)a.y, a.mean, a.rstd, a.N, plan.split,
                       plan.chunk_packs, a.eps);
    hipLaunchKernelGGL((norm_fwd_split_apply_kernel<T, WT, kStreamBlock, RMS, TY>), grid,
                       dim3(kStreamBlock), 0, stream, (const T*)a.x, res, (const WT*)a.gamma,
                       (const WT*)a.beta, h, (TY*)a.y, (const float*)a.mean,
                       (const float*)a.rstd, a.N, plan.chunk_packs);
  } else {
    hipLaunchKernelGGL((norm_fwd_stream_kernel<T, WT, kStreamBlock, RMS, TY>),
                       dim3((unsigned)plan.grid), dim3(kStreamBlock), 0, stream, (const T*)a.x,
                       res, (const WT*)a.gamma, (const WT*)a.beta, h, (TY*)a.y, a.mean, a.rstd,
                       a.M, a.N, a.eps);
  }
  return (int)hipGetLastError();
}

template <class T, class WT, bool RMS>
struct NormBwdCtx {
  const Plan& plan;
  const NormBwdArgs& a;
  hipStream_t stream;
};

template <class T, class WT, bool RMS, bool FAST, bool ADD>
struct NormBwdLauncher {
  template <int G, int V, int BLOCK>
  struct At {
    static bool run(const NormBwdCtx<T, WT, RMS>& c) {
      if constexpr (variant_built(OC_NORM_BWD, sizeof(T), G, V, FAST) &&
                    block_built(OC_NORM_BWD, G, BLOCK) &&
                    (!FAST || norm_bwd_instance_ok(sizeof(T), sizeof(WT), G, V, RMS, ADD))) {
        if (c.plan.G == G && c.plan.V == V && c.plan.block == BLOCK) {
          hipLaunchKernelGGL((norm_bwd_resident_kernel<T, WT, G, V, BLOCK, 1, RMS, FAST, ADD>),
                             dim3((unsigned)c.plan.grid), dim3(BLOCK), 0, c.stream,
                             (const T*)c.a.dy, (const T*)c.a.x, (const T*)c.a.dres, c.a.mean,
                             c.a.rstd, (const WT*)c.a.gamma, (T*)c.a.dx, c.a.part_dg,
                             c.a.part_db, c.a.M, c.a.N);
          return true;
        }
      }
      return false;
    }
  };
};

// The exact two-pack layouts (kNormBwdExact): entry I of the table, if the plan names it.
template <class T, class WT, bool RMS, bool ADD, int I>
inline bool launch_norm_bwd_exact_at(const Plan& plan, const NormBwdArgs& a, hipStream_t stream) {
  constexpr NormBwdExactLayout l = kNormBwdExact[I];
  if constexpr (sizeof(T) == 2 &&
                norm_bwd_exact_serves(l, !RMS, sizeof(WT) > sizeof(T), ADD)) {
    if (plan.G == l.G && plan.V == l.V && plan.block == l.block && plan.exact_depth == l.depth) {
      hipLaunchKernelGGL((norm_bwd_exact_kernel<T, WT, l.G, l.V, l.block, RMS, ADD, l.depth>),
                         dim3((unsigned)plan.grid), dim3(l.block), 0, stream, (const T*)a.dy,
                         (const T*)a.x, (const T*)a.dres, a.mean, a.rstd, (const WT*)a.gamma,
                         (T*)a.dx, a.part_dg, a.part_db, a.M, a.N);
      return true;
    }
  }
  return false;
}
template <class T, class WT, bool RMS, bool ADD, int... Is>
inline bool launch_norm_bwd_exact(const Plan& plan, const NormBwdArgs& a, hipStream_t stream,
                                  ilist<Is...>) {
  return (launch_norm_bwd_exact_at<T, WT, RMS, ADD, Is>(plan, a, stream) || ...);
}

// Backward of short ragged rows through LDS (norm_bwd_flat_kernel): two tensors of a piece
// in 16 KB each, 32 KB each for rows beyond 1024 16-bit elements.  The grid walks the pieces
// with a stride, as many workgroups as the plan has partial rows (the size of the caller's
// workspace); `*rows_out` receives how many partial rows the launch fills.
// 16-bit rows take it on up to 8 lanes a row (24 packs, 192 elements), fp32 rows at every
// length it covers: with 8 elements a pack the lane's gy / xhat / dgamma / dbeta registers are
// twice the fp32 kernel's and the general kernel wins from 16 lanes on.  131072 rows, LayerNorm /
// RMSNorm in us, general kernel -> this one: bf16 N = 17 31.7 / 24.7 -> 13.8 / 13.5, 100 42.6 /
// 36.9 -> 28.6 / 27.3, 127 54.1 / 48.8 -> 35.6 / 34.6, 150 54.3 / 48.7 -> 49.1 / 45.9, 257 (16
// lanes) 74.0 / 67.0 -> 85.1 / 76.8, 1001 169 / 163 -> 203 / 202; fp32 N = 17 30.6 / 23.0 -> 16.3 /
// 15.2, 63 47.2 / 41.4 -> 27.7 / 27.1, 127 78.9 / 74.1 -> 45.3 / 44.0, 257 96.2 / 90.9 -> 94.9 /
// 92.4, 1001 329 / 323 -> 312 / 306.  More workgroups than the plan's partial rows (3, 4 or 8 a
// compute unit instead of 2) measured slower at most lengths.
// Rows of whole packs (which the resident kernel addresses without conditions) only up to 64
// bytes, 32 in fp32: bf16 N = 8 80 -> 32 us, 16 45 -> 30, 32 31 -> 29 but 72 30 -> 40, 96 28 -> 34;
// fp32 N = 4 116 -> 53, 8 66 -> 54 but 16 44 -> 54 (2097152 / 1048576 / ... rows, LayerNorm).
constexpr bool norm_bwd_flat_serves(size_t esize, int lanes) { return esize == 4 || lanes <= 8; }
constexpr bool norm_bwd_flat_serves_whole_packs(size_t esize, int N) {
  return (size_t)N * esize <= (esize == 4 ? 32u : 64u);
}
template <class T, class WT, bool RMS, int LDSB>
bool launch_norm_bwd_flat_l(const Plan& plan, FlatLayout f, int cr, const NormBwdArgs& a,
                            hipStream_t stream, int* rows_out) {
  const int64_t pieces = (a.M + cr - 1) / cr;
  const int64_t cap = a.part_dg != nullptr ? (int64_t)plan.partial_rows : (int64_t)0x7fffffff;
  const int64_t grid = pieces < cap ? pieces : cap;
  if (grid < 1) return false;
#define ROWNORM_FLAT_NORM_BWD(GL, VP)                                                           \
  case GL * 8 + VP:                                                                             \
    if constexpr ((LDSB <= kFlatLdsBytes || (GL == 64 && VP >= 3)) &&                           \
                  norm_bwd_flat_serves(sizeof(T), GL)) {                                        \
      hipLaunchKernelGGL((norm_bwd_flat_kernel<T, WT, GL, VP, kFlatBlock, LDSB, RMS>),           \
                         dim3((unsigned)grid), dim3(kFlatBlock), 0, stream, (const T*)a.dy,      \
                         (const T*)a.x, a.mean, a.rstd, (const WT*)a.gamma, (T*)a.dx, a.part_dg, \
                         a.part_db, a.M, a.N, cr);                                              \
      *rows_out = (int)grid;                                                                    \
      return true;                                                                              \
    }                                                                                           \
    return false;
  switch (f.g * 8 + f.vp) { ROWNORM_FLAT_ALL(ROWNORM_FLAT_NORM_BWD) }
#undef ROWNORM_FLAT_NORM_BWD
  return false;
}

template <class T, class WT, bool RMS>
bool launch_norm_bwd_flat(const Plan& plan, FlatLayout f, const NormBwdArgs& a, hipStream_t stream,
                          int* rows_out) {
  int cr = flat_chunk_rows<T>(a.N, f.g, kFlatLdsBytes);
  if (cr >= 8)
    return launch_norm_bwd_flat_l<T, WT, RMS, kFlatLdsBytes>(plan, f, cr, a, stream, rows_out);
  cr = flat_chunk_rows<T>(a.N, f.g, 2 * kFlatLdsBytes);
  if (cr >= 8)
    return launch_norm_bwd_flat_l<T, WT, RMS, 2 * kFlatLdsBytes>(plan, f, cr, a, stream, rows_out);
  return false;
}

template <class T, class WT, bool RMS, bool ADD>
int launch_norm_bwd(const Plan& plan, const NormBwdArgs& a, hipStream_t stream) {
  const bool want_cols = a.part_dg != nullptr;
  const T* dres = ADD ? (const T*)a.dres : nullptr;
  int partial_rows = (int)plan.partial_rows;
  // one partial row (few, very long rows): the column-sum kernels write dgamma / dbeta themselves
  const bool team_call = !ADD && !plan.resident && plan.team > 0 && a.team_slot != nullptr && a.dx != nullptr;
  const bool direct = want_cols && !plan.resident && plan.partial_rows == 1 && !team_call;
  bool flat = false;
  // short ragged rows (no residual gradient, 16-byte aligned dY, X and dX): staged through LDS
  if constexpr (!ADD) {
    if (plan.resident && plan.exact_depth == 0 && !plan.window) {
      const FlatLayout f = flat_layout<T>(plan, a.M, a.N, a.dy, a.x, a.dx);
      flat = f.g != 0 && norm_bwd_flat_serves(sizeof(T), f.g) &&
             (!plan.fast || norm_bwd_flat_serves_whole_packs(sizeof(T), a.N)) &&
             launch_norm_bwd_flat<T, WT, RMS>(plan, f, a, stream, &partial_rows);
    }
  }
  if (flat) {
    // (launched above)
  } else if (plan.resident && plan.exact_depth > 0) {
    static_assert(kNormBwdExactCount == 15, "one index per table entry below");
    if (a.dx == nullptr || !launch_norm_bwd_exact<T, WT, RMS, ADD>(
                               plan, a, stream, ilist<0, 1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 11, 12, 13, 14>{}))
      return (int)hipErrorInvalidConfiguration;
  } else if (plan.resident) {
    NormBwdCtx<T, WT, RMS> ctx{plan, a, stream};
    const bool launched =
        plan.fast ? launch_variant<NormBwdLauncher<T, WT, RMS, true, ADD>::template At>(ctx)
                  : launch_variant<NormBwdLauncher<T, WT, RMS, false, ADD>::template At>(ctx);
    if (!launched) return (int)hipErrorInvalidConfiguration;
  } else if (team_call) {
    // rows beyond the registers, dY and X read once: teams of workgroups, one partial row each
    hipLaunchKernelGGL((norm_bwd_team_kernel<T, WT, RMS, kTeamBwdRows, kTeamBwdPacks>), dim3((unsigned)plan.team_grid),
                       dim3(kTeamBlock), 0, stream, (const T*)a.dy, (const T*)a.x, a.mean, a.rstd,
                       (const WT*)a.gamma, (T*)a.dx, a.part_dg, a.part_db, a.M, a.N, plan.team,
                       (TeamSlot*)a.team_slot, a.team_id, a.team_wait_ticks);
    partial_rows = (int)(plan.team_grid / plan.team);
  } else {
    constexpr int E = elems_per_pack<T>::value;
    bool cols_done = false;
    // the row sums s1, s2 go through memory when a row is split over workgroups,
    // and also when it is not but the column sums are wanted: dX and the column
    // sums then share the second pass over X and dY (two passes, not three)
    const int chunks = plan.split > 1 ? plan.split : 1;
    if (a.dx != nullptr && a.split_ws != nullptr && (chunks > 1 || want_cols) && a.M <= 65535) {
      const dim3 grid((unsigned)chunks, (unsigned)a.M);
      hipLaunchKernelGGL((norm_bwd_split_sums_kernel<T, WT, kStreamBlock, RMS>), grid,
                         dim3(kStreamBlock), 0, stream, (const T*)a.dy, (const T*)a.x, a.mean,
                         a.rstd, (const WT*)a.gamma, a.split_ws, a.N, plan.chunk_packs);
      if (want_cols) {
        // dX and the column sums in one more pass over X and dY
        constexpr int CB = 256;
        float* totals = a.split_ws;  // one chunk a row: its sums are the totals
        if (chunks > 1) {
          totals = a.split_ws + a.M * (int64_t)chunks * 2;
          hipLaunchKernelGGL((norm_bwd_split_totals_kernel<0>), dim3((unsigned)a.M), dim3(64), 0,
                             stream, (const float*)a.split_ws, totals, chunks);
        }
        const unsigned gx = (unsigned)((a.N + CB * E - 1) / (CB * E));
        hipLaunchKernelGGL((norm_bwd_split_dx_colsum_kernel<T, WT, CB, RMS>),
                           dim3(gx, (unsigned)plan.partial_rows), dim3(CB), 0, stream,
                           (const T*)a.dy, (const T*)a.x, dres, a.mean, a.rstd,
                           (const WT*)a.gamma, (const float*)totals, (T*)a.dx, a.part_dg,
                           a.part_db, (WT*)a.dgamma, (WT*)a.dbeta, (int)direct, a.M, a.N);
        cols_done = true;
      } else {
        hipLaunchKernelGGL((norm_bwd_split_dx_kernel<T, WT, kStreamBlock, RMS>), grid,
                           dim3(kStreamBlock), 0, stream, (const T*)a.dy, (const T*)a.x, dres,
                           a.mean, a.rstd, (const WT*)a.gamma, (const float*)a.split_ws,
                           (T*)a.dx, a.N, plan.chunk_packs);
      }
    } else if (a.dx != nullptr) {
      hipLaunchKernelGGL((norm_bwd_stream_dx_kernel<T, WT, kStreamBlock, RMS>),
                         dim3((unsigned)plan.grid), dim3(kStreamBlock), 0, stream,
                         (const T*)a.dy, (const T*)a.x, dres, a.mean, a.rstd,
                         (const WT*)a.gamma, (T*)a.dx, a.M, a.N);
    }
    if (want_cols && !cols_done) {
      constexpr int CB = 256;
      const unsigned gx = (unsigned)((a.N + CB * E - 1) / (CB * E));
      hipLaunchKernelGGL((norm_bwd_stream_colsum_kernel<T, WT, CB, RMS>),
                         dim3(gx, (unsigned)plan.partial_rows), dim3(CB), 0, stream,
                         (const T*)a.dy, (const T*)a.x, a.mean, a.rstd, a.part_dg, a.part_db,
                         (WT*)a.dgamma, (WT*)a.dbeta, (int)direct, a.M, a.N);
    }
  }
  int err = (int)hipGetLastError();
  if (err != 0 || !want_cols || direct) return err;
  if (!plan.resident && partial_rows <= kFinalizeFlatRows) {
    const unsigned gx = (unsigned)((a.N + kFinalizeFlatCols - 1) / kFinalizeFlatCols);
    hipLaunchKernelGGL((colsum_finalize_flat_kernel<WT>), dim3(gx, RMS ? 1 : 2), dim3(256), 0,
                       stream, (const float*)a.part_dg, (const float*)a.part_db, (WT*)a.dgamma,
                       (WT*)a.dbeta, partial_rows, a.N);
    return (int)hipGetLastError();
  }
  const unsigned gx = (unsigned)((a.N + kFinalizeCols - 1) / kFinalizeCols);
  hipLaunchKernelGGL((colsum_finalize_kernel<WT>), dim3(gx, RMS ? 1 : 2), dim3(1024), 0, stream,
                     (const float*)a.part_dg, (const float*)a.part_db, (WT*)a.dgamma,
                     (WT*)a.dbeta, partial_rows, a.N);
  return (int)hipGetLastError();
}

}  // namespace rownorm
