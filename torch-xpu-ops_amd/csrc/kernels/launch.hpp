// Typed launch entry points shared by the per-dtype translation units and the
// C ABI file.  Each launch_* template is defined in *_launch.hpp and explicitly
// instantiated in one of the *.hip files, so the kernels compile in parallel.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include "device/pack.hpp"
#include "plan.hpp"

namespace rownorm {

struct NormFwdArgs {
  const void* x;
  const void* gamma;
  const void* beta;
  void* y;
  float* mean;
  float* rstd;
  int64_t M;
  int N;
  float eps;
  // fused residual add: the row that is normalized is h = x + res, written to h
  // (both null: plain norm of x)
  const void* res = nullptr;
  void* h = nullptr;
  // norm_fwd_team_kernel: its slot of bookkeeping memory (null: that kernel is not
  // used), the id of this call and the bound of its waits in ticks of the
  // constant-rate clock
  void* team_slot = nullptr;
  unsigned int team_id = 0;
  unsigned long long team_wait_ticks = 0;
};

struct NormBwdArgs {
  const void* dy;
  const void* x;
  const float* mean;
  const float* rstd;
  const void* gamma;
  void* dx;
  void* dgamma;
  void* dbeta;
  float* part_dg;  // [plan.partial_rows, N] fp32, or null when no column sums are wanted
  float* part_db;
  int64_t M;
  int N;
  float* split_ws = nullptr;  // [M, plan.split + 1, 2] fp32 for the split-row path, or null: not split
  const void* dres = nullptr;  // gradient reaching the normalized row by the residual path, added to dx
  // norm_bwd_team_kernel (rows beyond the registers held by teams of workgroups): the call's
  // slot of bookkeeping memory, its id and the bound of a wait, as in NormFwdArgs; null = not
  // for this call.  part_dg / part_db then hold plan.team_partial_rows rows.
  void* team_slot = nullptr;
  unsigned int team_id = 0;
  unsigned long long team_wait_ticks = 0;
};

constexpr int kSoftmaxLog = 1;   // log_softmax instead of softmax
constexpr int kSoftmaxSafe = 2;  // rows with no finite element give 0 instead of NaN

struct SoftmaxFwdArgs {
  const void* x;
  void* y;
  const uint8_t* mask;  // null = unmasked; else data row r uses mask row (r / div) * stride + r % mod
  uint32_t mask_div, mask_mod;
  int64_t mask_stride;
  int64_t M;
  int N;
  int flags;  // kSoftmaxLog | kSoftmaxSafe
  // few very long rows held by teams of workgroups (softmax_fwd_team_kernel): the call's
  // slot of bookkeeping memory, its id and the bound of a wait; null = not for this call
  void* team_slot = nullptr;
  unsigned int team_id = 0;
  unsigned long long team_wait_ticks = 0;
};

struct SoftmaxBwdArgs {
  const void* grad;
  const void* y;
  void* gi;
  const uint8_t* mask;
  uint32_t mask_div, mask_mod;
  int64_t mask_stride;
  int64_t M;
  int N;
  int flags;
  // few very long rows held by teams of workgroups (softmax_bwd_team_kernel), as in the forward
  void* team_slot = nullptr;
  unsigned int team_id = 0;
  unsigned long long team_wait_ticks = 0;
};

struct SoftmaxStridedFwdArgs {
  const void* x;
  void* y;
  int64_t outer;
  int D, inner;
  int flags;
};

struct SoftmaxStridedBwdArgs {
  const void* grad;
  const void* y;
  void* gi;
  int64_t outer;
  int D, inner;
  int flags;
};

// GroupNorm on [N, C, HxW] with C = groups * D: rows = N * groups rows of L = D * HxW.
struct GroupNormFwdArgs {
  const void* x;
  const void* gamma;
  const void* beta;
  void* y;
  void* mean;  // [rows], weight dtype
  void* rstd;
  int64_t rows;
  int L, HxW, D, groups;
  float eps;
  // bookkeeping memory, call id and wait bound of the team forward (see NormFwdArgs)
  void* team_slot = nullptr;
  unsigned int team_id = 0;
  unsigned long long team_wait_ticks = 0;
};

struct GroupNormBwdArgs {
  const void* dy;
  const void* x;
  const void* mean;
  const void* rstd;
  const void* gamma;
  void* dx;
  void* dgamma;
  void* dbeta;
  float* part_dg;  // [N, C] fp32 each; null when the call needs no channel sums
  float* part_db;
  int64_t rows;
  int L, HxW, D, groups;
  // gn_bwd_team_kernel (slabs beyond the registers held by teams of workgroups): workgroups a
  // slab and a channel, packs a lane of each tensor, workgroups launched; the call's slot of
  // bookkeeping memory, its id and the bound of a wait, as in GroupNormFwdArgs; team == 0 or
  // a null slot: not for this call
  int team = 0, team_wpc = 0, team_v = 0;
  int64_t team_grid = 0;
  void* team_slot = nullptr;
  unsigned int team_id = 0;
  unsigned long long team_wait_ticks = 0;
};

inline bool regions_disjoint(const void* a, int64_t abytes, const void* b, int64_t bbytes) {
  if (a == nullptr || b == nullptr) return true;
  const char* pa = (const char*)a;
  const char* pb = (const char*)b;
  return pa + abytes <= pb || pb + bbytes <= pa;
}

// All return 0 or a hipError_t value.
// TY: element type of y (T, or a 16-bit type for float32 rows); ADD: a.res / a.h
// are given (forward), a.dres is given (backward).
template <class T, class WT, bool RMS, class TY = T, bool ADD = false>
int launch_norm_fwd(const Plan& plan, const NormFwdArgs& a, hipStream_t stream);
template <class T, class WT, bool RMS, bool ADD = false>
int launch_norm_bwd(const Plan& plan, const NormBwdArgs& a, hipStream_t stream);
template <class TI, class TO>
int launch_softmax_fwd(const Plan& plan, const SoftmaxFwdArgs& a, hipStream_t stream);
template <class TG, class TO>
int launch_softmax_bwd(const Plan& plan, const SoftmaxBwdArgs& a, hipStream_t stream);

template <class T, class WT>
int launch_group_norm_fwd(const Plan& plan, const GroupNormFwdArgs& a, hipStream_t stream);
template <class T, class WT>
int launch_group_norm_bwd(const Plan& plan, const GroupNormBwdArgs& a, hipStream_t stream);
template <class TI, class TO>
int launch_softmax_strided_fwd(const StridedPlan& plan, const SoftmaxStridedFwdArgs& a,
                               hipStream_t stream);
template <class TG, class TO>
int launch_softmax_strided_bwd(const StridedPlan& plan, const SoftmaxStridedBwdArgs& a,
                               hipStream_t stream);

// Compile-time walk over every (G, V, BLOCK) a kernel family may be built for;
// L<G, V, BLOCK>::run(ctx) returns true when it matched the plan and launched.
template <int... Is>
struct ilist {};
using GList = ilist<8, 16, 32, 64, 128, 256, 512, 1024>;
using VList = ilist<1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 11, 12, 13, 14, 15, 16, 17, 18, 19, 20>;
using BList = ilist<256, 512, 1024>;

template <template <int, int, int> class L, class Ctx, int G, int V, int... Bs>
inline bool try_blocks(const Ctx& c, ilist<Bs...>) {
  return (L<G, V, Bs>::run(c) || ...);
}
template <template <int, int, int> class L, class Ctx, int G, int... Vs>
inline bool try_packs(const Ctx& c, ilist<Vs...>) {
  return (try_blocks<L, Ctx, G, Vs>(c, BList{}) || ...);
}
template <template <int, int, int> class L, class Ctx, int... Gs>
inline bool try_lanes(const Ctx& c, ilist<Gs...>) {
  return (try_packs<L, Ctx, Gs>(c, VList{}) || ...);
}
template <template <int, int, int> class L, class Ctx>
inline bool launch_variant(const Ctx& c) {
  return try_lanes<L, Ctx>(c, GList{});
}

}  // namespace rownorm
