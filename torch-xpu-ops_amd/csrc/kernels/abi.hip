// extern "C" surface of libmi355x_rownorm.so (declared in include/mi355x_rownorm.h).
// Validates arguments, picks the launch layout and forwards to the typed
// launch templates; allocates nothing and never synchronizes.
#include "../../../include/mi355x_rownorm.h"

#include <atomic>
#include "launch.hpp"

namespace rownorm {
// defined in the per-dtype translation units
extern template int launch_norm_fwd<float, float, false>(const Plan&, const NormFwdArgs&, hipStream_t);
extern template int launch_norm_fwd<float, float, true>(const Plan&, const NormFwdArgs&, hipStream_t);
extern template int launch_norm_fwd<f16, f16, false>(const Plan&, const NormFwdArgs&, hipStream_t);
extern template int launch_norm_fwd<f16, f16, true>(const Plan&, const NormFwdArgs&, hipStream_t);
extern template int launch_norm_fwd<f16, float, false>(const Plan&, const NormFwdArgs&, hipStream_t);
extern template int launch_norm_fwd<f16, float, true>(const Plan&, const NormFwdArgs&, hipStream_t);
extern template int launch_norm_fwd<bf16, bf16, false>(const Plan&, const NormFwdArgs&, hipStream_t);
extern template int launch_norm_fwd<bf16, bf16, true>(const Plan&, const NormFwdArgs&, hipStream_t);
extern template int launch_norm_fwd<bf16, float, false>(const Plan&, const NormFwdArgs&, hipStream_t);
extern template int launch_norm_fwd<bf16, float, true>(const Plan&, const NormFwdArgs&, hipStream_t);
extern template int launch_norm_bwd<float, float, false>(const Plan&, const NormBwdArgs&, hipStream_t);
extern template int launch_norm_bwd<float, float, true>(const Plan&, const NormBwdArgs&, hipStream_t);
extern template int launch_norm_bwd<f16, f16, false>(const Plan&, const NormBwdArgs&, hipStream_t);
extern template int launch_norm_bwd<f16, f16, true>(const Plan&, const NormBwdArgs&, hipStream_t);
extern template int launch_norm_bwd<f16, float, false>(const Plan&, const NormBwdArgs&, hipStream_t);
extern template int launch_norm_bwd<f16, float, true>(const Plan&, const NormBwdArgs&, hipStream_t);
extern template int launch_norm_bwd<bf16, bf16, false>(const Plan&, const NormBwdArgs&, hipStream_t);
extern template int launch_norm_bwd<bf16, bf16, true>(const Plan&, const NormBwdArgs&, hipStream_t);
extern template int launch_norm_bwd<bf16, float, false>(const Plan&, const NormBwdArgs&, hipStream_t);
extern template int launch_norm_bwd<bf16, float, true>(const Plan&, const NormBwdArgs&, hipStream_t);
extern template int launch_norm_fwd<bf16, bf16, false, bf16, true>(const Plan&, const NormFwdArgs&, hipStream_t);
extern template int launch_norm_bwd<bf16, bf16, false, true>(const Plan&, const NormBwdArgs&, hipStream_t);
extern template int launch_norm_fwd<bf16, bf16, true, bf16, true>(const Plan&, const NormFwdArgs&, hipStream_t);
extern template int launch_norm_bwd<bf16, bf16, true, true>(const Plan&, const NormBwdArgs&, hipStream_t);
extern template int launch_norm_fwd<bf16, float, false, bf16, true>(const Plan&, const NormFwdArgs&, hipStream_t);
extern template int launch_norm_bwd<bf16, float, false, true>(const Plan&, const NormBwdArgs&, hipStream_t);
extern template int launch_norm_fwd<bf16, float, true, bf16, true>(const Plan&, const NormFwdArgs&, hipStream_t);
extern template int launch_norm_bwd<bf16, float, true, true>(const Plan&, const NormBwdArgs&, hipStream_t);
extern template int launch_norm_fwd<f16, f16, false, f16, true>(const Plan&, const NormFwdArgs&, hipStream_t);
extern template int launch_norm_bwd<f16, f16, false, true>(const Plan&, const NormBwdArgs&, hipStream_t);
extern template int launch_norm_fwd<f16, f16, true, f16, true>(const Plan&, const NormFwdArgs&, hipStream_t);
extern template int launch_norm_bwd<f16, f16, true, true>(const Plan&, const NormBwdArgs&, hipStream_t);
extern template int launch_norm_fwd<f16, float, false, f16, true>(const Plan&, const NormFwdArgs&, hipStream_t);
extern template int launch_norm_bwd<f16, float, false, true>(const Plan&, const NormBwdArgs&, hipStream_t);
extern template int launch_norm_fwd<f16, float, true, f16, true>(const Plan&, const NormFwdArgs&, hipStream_t);
extern template int launch_norm_bwd<f16, float, true, true>(const Plan&, const NormBwdArgs&, hipStream_t);
extern template int launch_norm_fwd<float, float, false, float, true>(const Plan&, const NormFwdArgs&, hipStream_t);
extern template int launch_norm_bwd<float, float, false, true>(const Plan&, const NormBwdArgs&, hipStream_t);
extern template int launch_norm_fwd<float, float, true, float, true>(const Plan&, const NormFwdArgs&, hipStream_t);
extern template int launch_norm_bwd<float, float, true, true>(const Plan&, const NormBwdArgs&, hipStream_t);
extern template int launch_norm_fwd<float, float, false, bf16, false>(const Plan&, const NormFwdArgs&, hipStream_t);
extern template int launch_norm_fwd<float, float, true, bf16, false>(const Plan&, const NormFwdArgs&, hipStream_t);
extern template int launch_norm_fwd<float, float, false, bf16, true>(const Plan&, const NormFwdArgs&, hipStream_t);
extern template int launch_norm_fwd<float, float, true, bf16, true>(const Plan&, const NormFwdArgs&, hipStream_t);
extern template int launch_norm_fwd<float, float, false, f16, false>(const Plan&, const NormFwdArgs&, hipStream_t);
extern template int launch_norm_fwd<float, float, true, f16, false>(const Plan&, const NormFwdArgs&, hipStream_t);
extern template int launch_norm_fwd<float, float, false, f16, true>(const Plan&, const NormFwdArgs&, hipStream_t);
extern template int launch_norm_fwd<float, float, true, f16, true>(const Plan&, const NormFwdArgs&, hipStream_t);
extern template int launch_softmax_fwd<float, float>(const Plan&, const SoftmaxFwdArgs&, hipStream_t);
extern template int launch_softmax_fwd<f16, f16>(const Plan&, const SoftmaxFwdArgs&, hipStream_t);
extern template int launch_softmax_fwd<bf16, bf16>(const Plan&, const SoftmaxFwdArgs&, hipStream_t);
extern template int launch_softmax_fwd<f16, float>(const Plan&, const SoftmaxFwdArgs&, hipStream_t);
extern template int launch_softmax_bwd<float, float>(const Plan&, const SoftmaxBwdArgs&, hipStream_t);
extern template int launch_softmax_bwd<f16, f16>(const Plan&, const SoftmaxBwdArgs&, hipStream_t);
extern template int launch_softmax_bwd<bf16, bf16>(const Plan&, const SoftmaxBwdArgs&, hipStream_t);
extern template int launch_softmax_bwd<float, f16>(const Plan&, const SoftmaxBwdArgs&, hipStream_t);
extern template int launch_group_norm_fwd<float, float>(const Plan&, const GroupNormFwdArgs&, hipStream_t);
extern template int launch_group_norm_fwd<f16, f16>(const Plan&, const GroupNormFwdArgs&, hipStream_t);
extern template int launch_group_norm_fwd<f16, float>(const Plan&, const GroupNormFwdArgs&, hipStream_t);
extern template int launch_group_norm_fwd<bf16, bf16>(const Plan&, const GroupNormFwdArgs&, hipStream_t);
extern template int launch_group_norm_fwd<bf16, float>(const Plan&, const GroupNormFwdArgs&, hipStream_t);
extern template int launch_group_norm_bwd<float, float>(const Plan&, const GroupNormBwdArgs&, hipStream_t);
extern template int launch_group_norm_bwd<f16, f16>(const Plan&, const GroupNormBwdArgs&, hipStream_t);
extern template int launch_group_norm_bwd<f16, float>(const Plan&, const GroupNormBwdArgs&, hipStream_t);
extern template int launch_group_norm_bwd<bf16, bf16>(const Plan&, const GroupNormBwdArgs&, hipStream_t);
extern template int launch_group_norm_bwd<bf16, float>(const Plan&, const GroupNormBwdArgs&, hipStream_t);
extern template int launch_softmax_strided_fwd<float, float>(const StridedPlan&, const SoftmaxStridedFwdArgs&, hipStream_t);
extern template int launch_softmax_strided_fwd<f16, f16>(const StridedPlan&, const SoftmaxStridedFwdArgs&, hipStream_t);
extern template int launch_softmax_strided_fwd<bf16, bf16>(const StridedPlan&, const SoftmaxStridedFwdArgs&, hipStream_t);
extern template int launch_softmax_strided_fwd<f16, float>(const StridedPlan&, const SoftmaxStridedFwdArgs&, hipStream_t);
extern template int launch_softmax_strided_bwd<float, float>(const StridedPlan&, const SoftmaxStridedBwdArgs&, hipStream_t);
extern template int launch_softmax_strided_bwd<f16, f16>(const StridedPlan&, const SoftmaxStridedBwdArgs&, hipStream_t);
extern template int launch_softmax_strided_bwd<bf16, bf16>(const StridedPlan&, const SoftmaxStridedBwdArgs&, hipStream_t);
extern template int launch_softmax_strided_bwd<float, f16>(const StridedPlan&, const SoftmaxStridedBwdArgs&, hipStream_t);
}  // namespace rownorm

using namespace rownorm;

namespace {

constexpr int64_t kMaxN = int64_t(1) << 30;
constexpr int kMaxDevices = 64;

// Compute units per device, looked up once per device (0 = not yet known).
std::atomic<int> g_num_cus[kMaxDevices];

int current_num_cus() {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) {
    (void)hipGetLastError();
    return 256;
  }
  if (dev < 0 || dev >= kMaxDevices) return 256;
  int n = g_num_cus[dev].load(std::memory_order_relaxed);
  if (n > 0) return n;
  int v = 0;
  if (hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess ||
      v <= 0) {
    (void)hipGetLastError();
    v = 256;
  }
  g_num_cus[dev].store(v, std::memory_order_relaxed);
  return v;
}

// Forced variants for tests and tuning (process-global, see the header).  One
// 64-bit atomic per op holds the four fields, so a call that runs while another
// thread sets an override sees the old or the new variant, never a mix.
std::atomic<uint64_t> g_override_bits[ROWNORM_OP_COUNT];

uint64_t pack_override(const Override& o) {
  return (uint64_t)(uint16_t)(int16_t)o.G | ((uint64_t)(uint16_t)o.V << 16) |
         ((uint64_t)(uint16_t)o.block << 32) | ((uint64_t)(uint16_t)o.bpc << 48);
}

struct OverrideTable {
  Override operator[](int op) const {
    const uint64_t b = g_override_bits[op].load(std::memory_order_relaxed);
    Override o;
    o.G = (int16_t)(uint16_t)(b & 0xffff);
    o.V = (int)((b >> 16) & 0xffff);
    o.block = (int)((b >> 32) & 0xffff);
    o.bpc = (int)((b >> 48) & 0xffff);
    return o;
  }
};
const OverrideTable g_override;

// Device-resident scratch of mi355x_rms_norm_bwd_static: the fp32 partial rows of
// the dgamma reduction (and the split-row partial sums behind them) for callers
// that may not allocate.  Every GPU the library runs on holds its own copy of
// the array, at its own address, until the process ends.  The name below is a
// host-side stand-in only; host code uses the per-device address that
// hipGetSymbolAddress reports (static_scratch()).
constexpr size_t kStaticScratchBytes = size_t(32) << 20;
static __device__ __align__(256) __attribute__((used)) unsigned char scratch[kStaticScratchBytes];
std::atomic<void*> g_scratch_ptr[kMaxDevices];

// The current device's address of `scratch`, looked up once per device.
// Returns 0, a positive hipError_t, or ROWNORM_ERR_SHAPE for a device ordinal
// beyond the table.
int static_scratch(void** out) {
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return (int)e;
  if (dev < 0 || dev >= kMaxDevices) return ROWNORM_ERR_SHAPE;
  void* p = g_scratch_ptr[dev].load(std::memory_order_acquire);
  if (p == nullptr) {
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess) return (int)e;
    if (p == nullptr) return (int)hipErrorInvalidSymbol;
    g_scratch_ptr[dev].store(p, std::memory_order_release);
  }
  *out = p;
  return 0;
}

// Bookkeeping memory of norm_fwd_team_kernel (the workgroups' partial sums), one slot
// a call, slots handed out round-robin; per device, like `scratch`.  Zero at load and
// never cleared: every word a call reads is tagged with the call's id.
static __device__ __align__(256) __attribute__((used)) TeamSlot team_slots[kTeamSlots];
std::atomic<void*> g_team_ptr[kMaxDevices];
std::atomic<unsigned int> g_team_calls{0};
// Bound of a workgroup's wait for its team, in ticks of the 100 MHz constant-rate
// clock: one second unless mi355x_rownorm_set_team_wait_us() says otherwise.
std::atomic<unsigned long long> g_team_wait_ticks{100000000ull};

// The slot and id of a new call on the current device, or null when the team
// kernel is not to be used: the address is not known, or the stream is being
// captured (a replay would run with the id of the capture).
void* team_slot_for_call(hipStream_t stream, unsigned int* id) {
  hipStreamCaptureStatus st = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(stream, &st) != hipSuccess) {
    (void)hipGetLastError();
    return nullptr;
  }
  if (st != hipStreamCaptureStatusNone) return nullptr;
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return nullptr;
  void* p = g_team_ptr[dev].load(std::memory_order_acquire);
  if (p == nullptr) {
    if (hipGetSymbolAddress(&p, HIP_SYMBOL(team_slots)) != hipSuccess || p == nullptr) {
      (void)hipGetLastError();
      return nullptr;
    }
    g_team_ptr[dev].store(p, std::memory_order_release);
  }
  unsigned int n = g_team_calls.fetch_add(1, std::memory_order_relaxed) + 1;
  if (n == 0) n = g_team_calls.fetch_add(1, std::memory_order_relaxed) + 1;  // 0 tags nothing
  *id = n;
  return (char*)p + (size_t)(n % kTeamSlots) * sizeof(TeamSlot);
}

int esize_of(int dt) {
  switch (dt) {
    case ROWNORM_F32: return 4;
    case ROWNORM_F16: return 2;
    case ROWNORM_BF16: return 2;
  }
  return 0;
}

bool norm_dtypes_ok(int x, int w) {
  if (esize_of(x) == 0 || esize_of(w) == 0) return false;
  return w == x || (w == ROWNORM_F32);
}

OpClass class_of(int op) {
  switch (op) {
    case ROWNORM_OP_LAYER_NORM_FWD:
    case ROWNORM_OP_RMS_NORM_FWD: return OC_NORM_FWD;
    case ROWNORM_OP_LAYER_NORM_BWD:
    case ROWNORM_OP_RMS_NORM_BWD: return OC_NORM_BWD;
    case ROWNORM_OP_SOFTMAX_FWD: return OC_SOFTMAX_FWD;
    default: return OC_SOFTMAX_BWD;
  }
}

int shape_check(int64_t M, int64_t N) {
  if (M < 0 || N < 0 || N > kMaxN) return ROWNORM_ERR_SHAPE;
  return 0;
}

// res / h: the fused residual add (both null: plain norm of x).  yd: dtype of y.
template <bool RMS>
int norm_fwd(const void* x, const void* res, const void* gamma, const void* beta, void* h,
             void* y, float* mean, float* rstd, int64_t M, int64_t N, float eps, int xd, int wd,
             int yd, void* stream) {
  if (!norm_dtypes_ok(xd, wd) || esize_of(yd) == 0) return ROWNORM_ERR_DTYPE;
  if (!(yd == xd || xd == ROWNORM_F32)) return ROWNORM_ERR_DTYPE;  // only float32 rows are cast
  if (int e = shape_check(M, N)) return e;
  if (M == 0 || N == 0) return 0;
  if (!x || !y || (res != nullptr && h == nullptr)) return ROWNORM_ERR_NULL;
  const bool add = res != nullptr;
  Plan plan;
  const int op = RMS ? ROWNORM_OP_RMS_NORM_FWD : ROWNORM_OP_LAYER_NORM_FWD;
  uintptr_t bits = (uintptr_t)x | (uintptr_t)y;
  if (add) bits |= (uintptr_t)res | (uintptr_t)h;
  const bool off_line = (bits & 127u) != 0;
  if (int e = make_plan(OC_NORM_FWD, M, N, esize_of(xd), current_num_cus(), g_override[op],
                        false, &plan, false, !RMS, esize_of(wd) > esize_of(xd), off_line, add))
    return e;
  NormFwdArgs a{x, gamma, RMS ? nullptr : beta, y, RMS ? nullptr : mean, rstd, M, (int)N, eps};
  if (add) {
    a.res = res;
    a.h = h;
  }
  hipStream_t s = (hipStream_t)stream;
  // (not in place: a workgroup of the team kernel whose team does not come together
  // reads the whole row of X, which must then still be X)
  const uintptr_t xb = (uintptr_t)x, yb = (uintptr_t)y;
  const uintptr_t nbytes = (uintptr_t)M * (uintptr_t)N * (uintptr_t)esize_of(xd);
  const bool y_on_x = xb < yb + nbytes && yb < xb + nbytes;
  if (plan.team > 0 && !add && yd == xd && !y_on_x) {
    a.team_slot = team_slot_for_call(s, &a.team_id);
    a.team_wait_ticks = g_team_wait_ticks.load(std::memory_order_relaxed);
  }
  if (xd == ROWNORM_F32) {
    if (yd == ROWNORM_BF16)
      return add ? launch_norm_fwd<float, float, RMS, bf16, true>(plan, a, s)
                 : launch_norm_fwd<float, float, RMS, bf16, false>(plan, a, s);
    if (yd == ROWNORM_F16)
      return add ? launch_norm_fwd<float, float, RMS, f16, true>(plan, a, s)
                 : launch_norm_fwd<float, float, RMS, f16, false>(plan, a, s);
    return add ? launch_norm_fwd<float, float, RMS, float, true>(plan, a, s)
               : launch_norm_fwd<float, float, RMS>(plan, a, s);
  }
  if (xd == ROWNORM_F16) {
    if (wd == ROWNORM_F32)
      return add ? launch_norm_fwd<f16, float, RMS, f16, true>(plan, a, s)
                 : launch_norm_fwd<f16, float, RMS>(plan, a, s);
    return add ? launch_norm_fwd<f16, f16, RMS, f16, true>(plan, a, s)
               : launch_norm_fwd<f16, f16, RMS>(plan, a, s);
  }
  if (wd == ROWNORM_F32)
    return add ? launch_norm_fwd<bf16, float, RMS, bf16, true>(plan, a, s)
               : launch_norm_fwd<bf16, float, RMS>(plan, a, s);
  return add ? launch_norm_fwd<bf16, bf16, RMS, bf16, true>(plan, a, s)
             : launch_norm_fwd<bf16, bf16, RMS>(plan, a, s);
}

// Bytes of the [M, split, 2] fp32 partial sums of the split-row backward and the
// [M, 2] row totals behind them; rows that stay on one workgroup but not in its
// registers keep their [M, 2] row sums there when the column sums are wanted as
// well (dX and the column sums then share one pass over X and dY).  0: neither.
// Partial rows of column sums a backward call may leave: those of the launch the plan names
// and, where teams of workgroups may hold the rows instead, one a team.
size_t bwd_partial_rows(const Plan& plan) {
  return (size_t)(plan.partial_rows > plan.team_partial_rows ? plan.partial_rows
                                                             : plan.team_partial_rows);
}

size_t split_bytes(const Plan& plan, int64_t M, bool want_cols) {
  if (plan.resident) return 0;
  if (plan.split > 1) return (size_t)M * ((size_t)plan.split + 1) * 2 * sizeof(float);
  return want_cols ? (size_t)M * 2 * sizeof(float) : 0;
}

// The query does not know whether the call will write dX or add a residual
// gradient, and the launch layout (hence the partial rows) may depend on both:
// it returns what the largest of those calls needs.
size_t norm_bwd_workspace(int op, int64_t M, int64_t N, int xd, int wd, int nparts) {
  if (!norm_dtypes_ok(xd, wd) || shape_check(M, N) || M == 0 || N == 0) return 0;
  size_t most = 0;
  for (int variant = 0; variant < 4; ++variant) {
    const bool fused_add = (variant & 1) != 0, want_dx = (variant & 2) != 0;
    if (fused_add && !want_dx) continue;  // the residual gradient is added to dX
    Plan plan;
    if (make_plan(OC_NORM_BWD, M, N, esize_of(xd), current_num_cus(), g_override[op], nparts > 0,
                  &plan, false, op == ROWNORM_OP_LAYER_NORM_BWD, esize_of(wd) > esize_of(xd),
                  false, fused_add, false, want_dx))
      return 0;
    const size_t need = bwd_partial_rows(plan) * (size_t)N * sizeof(float) * (size_t)nparts +
                        split_bytes(plan, M, nparts > 0);
    if (need > most) most = need;
  }
  return most;
}

// dres: the gradient reaching the normalized row by the residual path, added to dx (or null).
template <bool RMS>
int norm_bwd(const void* dy, const void* x, const float* mean, const float* rstd,
             const void* gamma, void* dx, void* dgamma, void* dbeta, void* workspace,
             size_t workspace_bytes, int64_t M, int64_t N, int xd, int wd, void* stream,
             const void* dres = nullptr) {
  if (!norm_dtypes_ok(xd, wd)) return ROWNORM_ERR_DTYPE;
  if (int e = shape_check(M, N)) return e;
  if (M == 0 || N == 0) return 0;
  if (RMS) dbeta = nullptr;
  const bool want_cols = dgamma != nullptr || dbeta != nullptr;
  if (!dx && !want_cols) return 0;
  if (!dy || !x || !rstd || (!RMS && !mean)) return ROWNORM_ERR_NULL;
  Plan plan;
  const int op = RMS ? ROWNORM_OP_RMS_NORM_BWD : ROWNORM_OP_LAYER_NORM_BWD;
  if (int e = make_plan(OC_NORM_BWD, M, N, esize_of(xd), current_num_cus(), g_override[op],
                        want_cols, &plan, false, !RMS, esize_of(wd) > esize_of(xd), false,
                        dres != nullptr && dx != nullptr, false, dx != nullptr))
    return e;
  float* part_dg = nullptr;
  float* part_db = nullptr;
  size_t need = 0;
  if (want_cols) {
    const size_t one = bwd_partial_rows(plan) * (size_t)N * sizeof(float);
    need = one * (RMS ? 1 : 2);
    if (!workspace || workspace_bytes < need) return ROWNORM_ERR_WORKSPACE;
    part_dg = (float*)workspace;
    part_db = RMS ? nullptr : (float*)((char*)workspace + one);
  }
  NormBwdArgs a{dy, x, mean, rstd, gamma, dx, dgamma, dbeta, part_dg, part_db, M, (int)N};
  // the split-row dX takes its partial sums behind the column sums when the
  // caller brought the room for them; without it a row stays on one workgroup
  if (dx && workspace && split_bytes(plan, M, want_cols) > 0 &&
      workspace_bytes >= need + split_bytes(plan, M, want_cols))
    a.split_ws = (float*)((char*)workspace + need);
  hipStream_t s = (hipStream_t)stream;
  // rows beyond the registers: the team backward (whole packs on 16-byte aligned tensors, dX
  // apart from dY and X -- a workgroup whose team does not come together reads whole rows of
  // both while others write theirs)
  if (plan.team > 0 && dx && !dres &&
      ((((uintptr_t)dy) | ((uintptr_t)x) | ((uintptr_t)dx) | ((uintptr_t)gamma) |
        ((uintptr_t)workspace)) & 15u) == 0) {
    const size_t nbytes = (size_t)M * (size_t)N * (size_t)esize_of(xd);
    const char *db = (const char*)dx, *gb = (const char*)dy, *xb = (const char*)x;
    if (!(db < gb + nbytes && gb < db + nbytes) && !(db < xb + nbytes && xb < db + nbytes)) {
      a.team_slot = team_slot_for_call(s, &a.team_id);
      a.team_wait_ticks = g_team_wait_ticks.load(std::memory_order_relaxed);
    }
  }
  if (dres != nullptr && dx != nullptr) {
    a.dres = dres;
    if (xd == ROWNORM_F32) return launch_norm_bwd<float, float, RMS, true>(plan, a, s);
    if (xd == ROWNORM_F16)
      return wd == ROWNORM_F32 ? launch_norm_bwd<f16, float, RMS, true>(plan, a, s)
                               : launch_norm_bwd<f16, f16, RMS, true>(plan, a, s);
    return wd == ROWNORM_F32 ? launch_norm_bwd<bf16, float, RMS, true>(plan, a, s)
                             : launch_norm_bwd<bf16, bf16, RMS, true>(plan, a, s);
  }
  if (xd == ROWNORM_F32) return launch_norm_bwd<float, float, RMS>(plan, a, s);
  if (xd == ROWNORM_F16)
    return wd == ROWNORM_F32 ? launch_norm_bwd<f16, float, RMS>(plan, a, s)
                             : launch_norm_bwd<f16, f16, RMS>(plan, a, s);
  return wd == ROWNORM_F32 ? launch_norm_bwd<bf16, float, RMS>(plan, a, s)
                           : launch_norm_bwd<bf16, bf16, RMS>(plan, a, s);
}

// How the rows of a mask buffer map onto data rows: data row r reads mask row
// (r / div) * stride + r % mod of a [rows, N] byte buffer.
struct MaskRows {
  int64_t rows = 0, div = 1, stride = 0, mod = 1;
};

// Rejects a mapping that could index outside the mask buffer.
int mask_check(const MaskRows& m, int64_t data_rows) {
  if (data_rows >= (int64_t(1) << 31)) return ROWNORM_ERR_SHAPE;
  if (m.rows <= 0 || m.div <= 0 || m.mod <= 0 || m.stride < 0) return ROWNORM_ERR_SHAPE;
  if (m.div >= (int64_t(1) << 32) || m.mod >= (int64_t(1) << 32)) return ROWNORM_ERR_SHAPE;
  const int64_t last = data_rows - 1;
  const int64_t hi_outer = last / m.div;
  if (m.stride != 0 && hi_outer > (m.rows - 1) / m.stride) return ROWNORM_ERR_SHAPE;
  const int64_t hi_inner = last < m.mod - 1 ? last : m.mod - 1;
  if (hi_outer * m.stride + hi_inner > m.rows - 1) return ROWNORM_ERR_SHAPE;
  return 0;
}

int softmax_fwd(const void* x, const void* mask, void* y, int64_t rows, int64_t N,
                const MaskRows& mr, int id, int od, int flags, void* stream) {
  if (esize_of(id) == 0 || esize_of(od) == 0) return ROWNORM_ERR_DTYPE;
  if (!(od == id || (id == ROWNORM_F16 && od == ROWNORM_F32))) return ROWNORM_ERR_DTYPE;
  if (int e = shape_check(rows, N)) return e;
  if (rows == 0 || N == 0) return 0;
  if (!x || !y) return ROWNORM_ERR_NULL;
  if (mask)
    if (int e = mask_check(mr, rows)) return e;
  Plan plan;
  const bool off_line = (((uintptr_t)x | (uintptr_t)y) & 127u) != 0;
  if (int e = make_plan(OC_SOFTMAX_FWD, rows, N, esize_of(id), current_num_cus(),
                        g_override[ROWNORM_OP_SOFTMAX_FWD], false, &plan, false, false, false,
                        off_line, false, mask != nullptr))
    return e;
  SoftmaxFwdArgs a{x,    y, (const uint8_t*)mask, (uint32_t)mr.div, (uint32_t)mr.mod, mr.stride,
                   rows, (int)N, flags};
  hipStream_t s = (hipStream_t)stream;
  // few very long rows: the team forward (whole packs on 16-byte aligned tensors, no mask,
  // Y apart from X -- a workgroup whose team does not come together reads the whole row
  // again -- and no stream capture)
  if (plan.team > 0 && !mask && ((((uintptr_t)x) | ((uintptr_t)y)) & 15u) == 0) {
    const char* xb = (const char*)x;
    const char* yb = (const char*)y;
    const size_t xbytes = (size_t)rows * (size_t)N * (size_t)esize_of(id);
    const size_t ybytes = (size_t)rows * (size_t)N * (size_t)esize_of(od);
    if (!(xb < yb + ybytes && yb < xb + xbytes)) {
      a.team_slot = team_slot_for_call(s, &a.team_id);
      a.team_wait_ticks = g_team_wait_ticks.load(std::memory_order_relaxed);
    }
  }
  if (id == ROWNORM_F32) return launch_softmax_fwd<float, float>(plan, a, s);
  if (id == ROWNORM_BF16) return launch_softmax_fwd<bf16, bf16>(plan, a, s);
  return od == ROWNORM_F32 ? launch_softmax_fwd<f16, float>(plan, a, s)
                           : launch_softmax_fwd<f16, f16>(plan, a, s);
}

int softmax_bwd(const void* grad, const void* y, const void* mask, void* gi, int64_t rows,
                int64_t N, const MaskRows& mr, int gd, int od, int flags, void* stream) {
  if (esize_of(gd) == 0 || esize_of(od) == 0) return ROWNORM_ERR_DTYPE;
  if (!(od == gd || (gd == ROWNORM_F32 && od == ROWNORM_F16))) return ROWNORM_ERR_DTYPE;
  if (int e = shape_check(rows, N)) return e;
  if (rows == 0 || N == 0) return 0;
  if (!grad || !y || !gi) return ROWNORM_ERR_NULL;
  if (mask)
    if (int e = mask_check(mr, rows)) return e;
  Plan plan;
  const bool off_line = (((uintptr_t)grad | (uintptr_t)y | (uintptr_t)gi) & 127u) != 0;
  if (int e = make_plan(OC_SOFTMAX_BWD, rows, N, esize_of(gd), current_num_cus(),
                        g_override[ROWNORM_OP_SOFTMAX_BWD], false, &plan, false, false, false,
                        off_line, false, mask != nullptr))
    return e;
  SoftmaxBwdArgs a{grad, y, gi, (const uint8_t*)mask, (uint32_t)mr.div, (uint32_t)mr.mod,
                   mr.stride, rows, (int)N, flags};
  hipStream_t s = (hipStream_t)stream;
  // few very long rows: the team backward, under the rules of the forward (gi apart from
  // grad and y)
  if (plan.team > 0 && !mask &&
      ((((uintptr_t)grad) | ((uintptr_t)y) | ((uintptr_t)gi)) & 15u) == 0) {
    const char* ob = (const char*)gi;
    const size_t ibytes = (size_t)rows * (size_t)N * (size_t)esize_of(gd);
    const size_t obytes = (size_t)rows * (size_t)N * (size_t)esize_of(od);
    auto apart = [&](const void* in) {
      const char* ib = (const char*)in;
      return !(ib < ob + obytes && ob < ib + ibytes);
    };
    if (apart(grad) && apart(y)) {
      a.team_slot = team_slot_for_call(s, &a.team_id);
      a.team_wait_ticks = g_team_wait_ticks.load(std::memory_order_relaxed);
    }
  }
  if (gd == ROWNORM_BF16) return launch_softmax_bwd<bf16, bf16>(plan, a, s);
  if (gd == ROWNORM_F16) return launch_softmax_bwd<f16, f16>(plan, a, s);
  return od == ROWNORM_F16 ? launch_softmax_bwd<float, f16>(plan, a, s)
                           : launch_softmax_bwd<float, float>(plan, a, s);
}

// Shape of a GroupNorm call as the kernels see it; returns 0 or an error code.
struct GroupDims {
  int64_t rows = 0;  // N * groups
  int64_t L = 0;     // (C / groups) * HxW
  int64_t D = 0;
};

int group_dims(int64_t N, int64_t C, int64_t HxW, int64_t groups, GroupDims* out) {
  if (N < 0 || C < 0 || HxW < 0 || groups <= 0) return ROWNORM_ERR_SHAPE;
  if (C % groups != 0) return ROWNORM_ERR_SHAPE;
  GroupDims d;
  d.D = C / groups;
  if (C >= (int64_t(1) << 31) || HxW > kMaxN || d.D > kMaxN) return ROWNORM_ERR_SHAPE;
  d.L = d.D * HxW;
  if (d.L > kMaxN) return ROWNORM_ERR_SHAPE;
  if (N >= (int64_t(1) << 31) / groups) return ROWNORM_ERR_SHAPE;
  d.rows = N * groups;
  *out = d;
  return 0;
}

// The general kernels are taken when neither every pack lies in one channel nor
// the straddling kernels apply (gn_mode, plan.hpp).
int group_plan(OpClass oc, int op, const GroupDims& d, int64_t HxW, int esize, Plan* plan,
               bool want_dx = true) {
  const int E = 16 / esize;
  const Override& ov = g_override[op];
  const int num_cus = current_num_cus();
  if (int e = make_plan(oc, d.rows, d.L, esize, num_cus, ov, false, plan,
                        gn_mode(d.L, HxW, d.D, E) == kGnGeneral))
    return e;
  // 16-bit rows that fill an exact layout and whose channels are whole runs of 64 packs
  const bool backward = oc == OC_GROUP_BWD;
  if (plan->resident && plan->fast && !plan->forced && ov.bpc == 0 && (want_dx || !backward)) {
    const int xi = group_exact_index(backward, esize, d.rows, d.L, HxW, d.D);
    if (xi >= 0) {
      const GroupExactLayout& l = kGroupExact[xi];
      plan->G = plan->block = l.G;
      plan->V = l.V;
      plan->rpb = 1;
      plan->exact_depth = 1;
      const int64_t cap = (int64_t)num_cus * (backward ? l.bpc_bwd : l.bpc_fwd);
      plan->grid = d.rows < cap ? d.rows : cap;
    }
  }
  return 0;
}

int softmax_mode_flags(int mode, bool forward, int* flags) {
  switch (mode) {
    case ROWNORM_SOFTMAX: *flags = 0; return 0;
    case ROWNORM_LOG_SOFTMAX: *flags = kSoftmaxLog; return 0;
    case ROWNORM_SAFE_SOFTMAX:
      if (!forward) break;  // its backward is the plain softmax backward
      *flags = kSoftmaxSafe;
      return 0;
  }
  return ROWNORM_ERR_SHAPE;
}

int strided_shape_check(int64_t outer, int64_t D, int64_t inner) {
  if (outer < 0 || D < 0 || inner < 0 || D > kMaxN || inner > kMaxN) return ROWNORM_ERR_SHAPE;
  return 0;
}

}  // namespace

extern "C" {

const char* mi355x_rownorm_error_string(int code) {
  switch (code) {
    case ROWNORM_OK: return "success";
    case ROWNORM_ERR_DTYPE: return "mi355x_rownorm: unsupported dtype or dtype pair";
    case ROWNORM_ERR_SHAPE: return "mi355x_rownorm: invalid shape (negative size or N > 2^30)";
    case ROWNORM_ERR_NULL: return "mi355x_rownorm: a required pointer is NULL";
    case ROWNORM_ERR_WORKSPACE: return "mi355x_rownorm: workspace missing or too small";
    case ROWNORM_ERR_OVERRIDE: return "mi355x_rownorm: forced variant cannot run this shape";
    case ROWNORM_ERR_SCRATCH_LIMIT:
      return "mi355x_rownorm: the call needs more scratch than the library's static 32 MiB";
  }
  if (code > 0) return hipGetErrorString((hipError_t)code);
  return "mi355x_rownorm: unknown error code";
}

int mi355x_rownorm_abi_version(void) { return 1; }

int mi355x_layer_norm_fwd(const void* x, const void* gamma, const void* beta, void* y,
                          float* mean, float* rstd, int64_t M, int64_t N, float eps,
                          rownorm_dtype x_dtype, rownorm_dtype w_dtype, void* stream) {
  return norm_fwd<false>(x, nullptr, gamma, beta, nullptr, y, mean, rstd, M, N, eps, (int)x_dtype,
                         (int)w_dtype, (int)x_dtype, stream);
}

int mi355x_add_layer_norm_fwd(const void* x, const void* residual, const void* gamma,
                              const void* beta, void* h, void* y, float* mean, float* rstd,
                              int64_t M, int64_t N, float eps, rownorm_dtype x_dtype,
                              rownorm_dtype w_dtype, rownorm_dtype y_dtype, void* stream) {
  return norm_fwd<false>(x, residual, gamma, beta, h, y, mean, rstd, M, N, eps, (int)x_dtype,
                         (int)w_dtype, (int)y_dtype, stream);
}

int mi355x_add_rms_norm_fwd(const void* x, const void* residual, const void* gamma, void* h,
                            void* y, float* rstd, int64_t M, int64_t N, float eps,
                            rownorm_dtype x_dtype, rownorm_dtype w_dtype, rownorm_dtype y_dtype,
                            void* stream) {
  return norm_fwd<true>(x, residual, gamma, nullptr, h, y, nullptr, rstd, M, N, eps,
                        (int)x_dtype, (int)w_dtype, (int)y_dtype, stream);
}

int mi355x_add_layer_norm_bwd(const void* dy, const void* dh_in, const void* h, const float* mean,
                              const float* rstd, const void* gamma, void* dh, void* dgamma,
                              void* dbeta, void* workspace, size_t workspace_bytes, int64_t M,
                              int64_t N, rownorm_dtype x_dtype, rownorm_dtype w_dtype,
                              void* stream) {
  return norm_bwd<false>(dy, h, mean, rstd, gamma, dh, dgamma, dbeta, workspace, workspace_bytes,
                         M, N, (int)x_dtype, (int)w_dtype, stream, dh_in);
}

int mi355x_add_rms_norm_bwd(const void* dy, const void* dh_in, const void* h, const float* rstd,
                            const void* gamma, void* dh, void* dgamma, void* workspace,
                            size_t workspace_bytes, int64_t M, int64_t N, rownorm_dtype x_dtype,
                            rownorm_dtype w_dtype, void* stream) {
  return norm_bwd<true>(dy, h, nullptr, rstd, gamma, dh, dgamma, nullptr, workspace,
                        workspace_bytes, M, N, (int)x_dtype, (int)w_dtype, stream, dh_in);
}

int mi355x_rms_norm_fwd(const void* x, const void* gamma, void* y, float* rstd, int64_t M,
                        int64_t N, float eps, rownorm_dtype x_dtype, rownorm_dtype w_dtype,
                        void* stream) {
  return norm_fwd<true>(x, nullptr, gamma, nullptr, nullptr, y, nullptr, rstd, M, N, eps,
                        (int)x_dtype, (int)w_dtype, (int)x_dtype, stream);
}

size_t mi355x_layer_norm_bwd_workspace_bytes(int64_t M, int64_t N, rownorm_dtype x_dtype,
                                             rownorm_dtype w_dtype, int want_dgamma,
                                             int want_dbeta) {
  return norm_bwd_workspace(ROWNORM_OP_LAYER_NORM_BWD, M, N, (int)x_dtype, (int)w_dtype,
                            (want_dgamma || want_dbeta) ? 2 : 0);
}

size_t mi355x_rms_norm_bwd_workspace_bytes(int64_t M, int64_t N, rownorm_dtype x_dtype,
                                           rownorm_dtype w_dtype, int want_dgamma) {
  return norm_bwd_workspace(ROWNORM_OP_RMS_NORM_BWD, M, N, (int)x_dtype, (int)w_dtype,
                            want_dgamma ? 1 : 0);
}

int mi355x_layer_norm_bwd(const void* dy, const void* x, const float* mean, const float* rstd,
                          const void* gamma, void* dx, void* dgamma, void* dbeta,
                          void* workspace, size_t workspace_bytes, int64_t M, int64_t N,
                          rownorm_dtype x_dtype, rownorm_dtype w_dtype, void* stream) {
  return norm_bwd<false>(dy, x, mean, rstd, gamma, dx, dgamma, dbeta, workspace, workspace_bytes,
                         M, N, (int)x_dtype, (int)w_dtype, stream);
}

int mi355x_rms_norm_bwd(const void* dy, const void* x, const float* rstd, const void* gamma,
                        void* dx, void* dgamma, void* workspace, size_t workspace_bytes,
                        int64_t M, int64_t N, rownorm_dtype x_dtype, rownorm_dtype w_dtype,
                        void* stream) {
  return norm_bwd<true>(dy, x, nullptr, rstd, gamma, dx, dgamma, nullptr, workspace,
                        workspace_bytes, M, N, (int)x_dtype, (int)w_dtype, stream);
}

size_t mi355x_rms_norm_bwd_static_limit_bytes(void) { return kStaticScratchBytes; }

int mi355x_rms_norm_bwd_static(const void* dy, const void* x, const float* rstd,
                               const void* gamma, void* dx, void* dgamma, int64_t M, int64_t N,
                               rownorm_dtype x_dtype, rownorm_dtype w_dtype, void* stream) {
  if (!norm_dtypes_ok((int)x_dtype, (int)w_dtype)) return ROWNORM_ERR_DTYPE;
  if (int e = shape_check(M, N)) return e;
  if (M == 0 || N == 0 || (!dx && !dgamma)) return 0;
  // What the allocating entry point would be given in full: the column-sum
  // partial rows and, for a few very long rows, the split-row partial sums.
  const size_t need = norm_bwd_workspace(ROWNORM_OP_RMS_NORM_BWD, M, N, (int)x_dtype,
                                         (int)w_dtype, dgamma ? 1 : 0);
  if (need > kStaticScratchBytes) return ROWNORM_ERR_SCRATCH_LIMIT;
  void* ws = nullptr;
  if (need > 0)
    if (int e = static_scratch(&ws)) return e;
  return norm_bwd<true>(dy, x, nullptr, rstd, gamma, dx, dgamma, nullptr, ws, need, M, N,
                        (int)x_dtype, (int)w_dtype, stream);
}

int mi355x_softmax_fwd(const void* x, void* y, int64_t rows, int64_t N, rownorm_dtype in_dtype,
                       rownorm_dtype out_dtype, int is_log, void* stream) {
  return softmax_fwd(x, nullptr, y, rows, N, MaskRows{}, (int)in_dtype, (int)out_dtype,
                     is_log ? kSoftmaxLog : 0, stream);
}

int mi355x_safe_softmax_fwd(const void* x, void* y, int64_t rows, int64_t N,
                            rownorm_dtype in_dtype, rownorm_dtype out_dtype, void* stream) {
  return softmax_fwd(x, nullptr, y, rows, N, MaskRows{}, (int)in_dtype, (int)out_dtype,
                     kSoftmaxSafe, stream);
}

int mi355x_masked_softmax_fwd(const void* x, const void* mask, void* y, int64_t rows, int64_t N,
                              int64_t mask_rows, int64_t mask_row_div, int64_t mask_row_stride,
                              int64_t mask_row_mod, rownorm_dtype dtype, void* stream) {
  if (rows > 0 && N > 0 && !mask) return ROWNORM_ERR_NULL;
  return softmax_fwd(x, mask, y, rows, N,
                     MaskRows{mask_rows, mask_row_div, mask_row_stride, mask_row_mod}, (int)dtype,
                     (int)dtype, 0, stream);
}

int mi355x_softmax_bwd(const void* grad, const void* y, void* gi, int64_t rows, int64_t N,
                       rownorm_dtype grad_dtype, rownorm_dtype gi_dtype, int is_log,
                       void* stream) {
  return softmax_bwd(grad, y, nullptr, gi, rows, N, MaskRows{}, (int)grad_dtype, (int)gi_dtype,
                     is_log ? kSoftmaxLog : 0, stream);
}

int mi355x_masked_softmax_bwd(const void* grad, const void* y, const void* mask, void* gi,
                              int64_t rows, int64_t N, int64_t mask_rows, int64_t mask_row_div,
                              int64_t mask_row_stride, int64_t mask_row_mod, rownorm_dtype dtype,
                              void* stream) {
  if (rows > 0 && N > 0 && !mask) return ROWNORM_ERR_NULL;
  return softmax_bwd(grad, y, mask, gi, rows, N,
                     MaskRows{mask_rows, mask_row_div, mask_row_stride, mask_row_mod}, (int)dtype,
                     (int)dtype, 0, stream);
}

int mi355x_group_norm_fwd(const void* x, const void* gamma, const void* beta, void* y, void* mean,
                          void* rstd, int64_t N, int64_t C, int64_t HxW, int64_t groups, float eps,
                          rownorm_dtype x_dtype, rownorm_dtype w_dtype, void* stream) {
  const int xd = (int)x_dtype, wd = (int)w_dtype;
  if (!norm_dtypes_ok(xd, wd)) return ROWNORM_ERR_DTYPE;
  GroupDims d;
  if (int e = group_dims(N, C, HxW, groups, &d)) return e;
  if (d.rows == 0 || d.L == 0) return 0;
  if (!x || !y) return ROWNORM_ERR_NULL;
  Plan plan;
  if (int e = group_plan(OC_GROUP_FWD, ROWNORM_OP_GROUP_NORM_FWD, d, HxW, esize_of(xd), &plan))
    return e;
  GroupNormFwdArgs a{x,      gamma,      beta,     y,          mean,        rstd,
                     d.rows, (int)d.L, (int)HxW, (int)d.D, (int)groups, eps};
  hipStream_t s = (hipStream_t)stream;
  // slabs beyond the registers: the team forward, under the rules of the norm forward
  // (not on top of X, not on a stream under capture)
  const uintptr_t xb = (uintptr_t)x, yb = (uintptr_t)y;
  const uintptr_t nbytes = (uintptr_t)d.rows * (uintptr_t)d.L * (uintptr_t)esize_of(xd);
  if (plan.team > 0 && !(xb < yb + nbytes && yb < xb + nbytes)) {
    a.team_slot = team_slot_for_call(s, &a.team_id);
    a.team_wait_ticks = g_team_wait_ticks.load(std::memory_order_relaxed);
  }
  if (xd == ROWNORM_F32) return launch_group_norm_fwd<float, float>(plan, a, s);
  if (xd == ROWNORM_F16)
    return wd == ROWNORM_F32 ? launch_group_norm_fwd<f16, float>(plan, a, s)
                             : launch_group_norm_fwd<f16, f16>(plan, a, s);
  return wd == ROWNORM_F32 ? launch_group_norm_fwd<bf16, float>(plan, a, s)
                           : launch_group_norm_fwd<bf16, bf16>(plan, a, s);
}

size_t mi355x_group_norm_bwd_workspace_bytes(int64_t N, int64_t C, int64_t HxW, int64_t groups,
                                             rownorm_dtype x_dtype, rownorm_dtype w_dtype,
                                             int want_dgamma, int want_dbeta) {
  GroupDims d;
  if (!norm_dtypes_ok((int)x_dtype, (int)w_dtype) || group_dims(N, C, HxW, groups, &d)) return 0;
  if (d.rows == 0 || d.L == 0) return 0;
  if (!(want_dgamma || want_dbeta)) {
    // rows too long for the registers compute dX from the channel sums
    Plan plan;
    if (group_plan(OC_GROUP_BWD, ROWNORM_OP_GROUP_NORM_BWD, d, HxW, esize_of((int)x_dtype), &plan))
      return 0;
    if (plan.resident) return 0;
  }
  return (size_t)N * (size_t)C * sizeof(float) * 2;
}

int mi355x_group_norm_bwd(const void* dy, const void* x, const void* mean, const void* rstd,
                          const void* gamma, void* dx, void* dgamma, void* dbeta, void* workspace,
                          size_t workspace_bytes, int64_t N, int64_t C, int64_t HxW,
                          int64_t groups, rownorm_dtype x_dtype, rownorm_dtype w_dtype,
                          void* stream) {
  const int xd = (int)x_dtype, wd = (int)w_dtype;
  if (!norm_dtypes_ok(xd, wd)) return ROWNORM_ERR_DTYPE;
  GroupDims d;
  if (int e = group_dims(N, C, HxW, groups, &d)) return e;
  if (d.rows == 0 || d.L == 0) return 0;
  const bool want_cols = dgamma != nullptr || dbeta != nullptr;
  if (!dx && !want_cols) return 0;
  if (!dy || !x || !mean || !rstd) return ROWNORM_ERR_NULL;
  Plan plan;
  if (int e = group_plan(OC_GROUP_BWD, ROWNORM_OP_GROUP_NORM_BWD, d, HxW, esize_of(xd), &plan,
                         dx != nullptr))
    return e;
  float* part_dg = nullptr;
  float* part_db = nullptr;
  if (want_cols || (!plan.resident && dx)) {
    const size_t one = (size_t)N * (size_t)C * sizeof(float);
    if (!workspace || workspace_bytes < 2 * one) return ROWNORM_ERR_WORKSPACE;
    part_dg = (float*)workspace;
    part_db = (float*)((char*)workspace + one);
  }
  GroupNormBwdArgs a{dy,      x,       mean,   rstd,     gamma,    dx,       dgamma,     dbeta,
                     part_dg, part_db, d.rows, (int)d.L, (int)HxW, (int)d.D, (int)groups};
  hipStream_t s = (hipStream_t)stream;
  // slabs beyond the registers whose channels are whole packs, 16-byte aligned tensors, dX
  // apart from dY and X (a workgroup whose team does not come together reads the whole slab
  // of both while others write theirs): teams of workgroups, dY and X read once.  As few
  // packs a lane (4 or 8 of each tensor) as hold a channel on one workgroup, else 8 and
  // several workgroups a channel, the last of them at least half full.
  const int64_t E = 16 / esize_of(xd);
  if (!plan.resident && dx && HxW % E == 0 &&
      ((((uintptr_t)dy) | ((uintptr_t)x) | ((uintptr_t)dx)) & 15u) == 0) {
    const size_t nbytes = (size_t)d.rows * (size_t)d.L * (size_t)esize_of(xd);
    const char *ob = (const char*)dx, *gb = (const char*)dy, *xb = (const char*)x;
    const int64_t cp = HxW / E;
    int v = 8;
    for (int t = 1; t < 8; t *= 2)
      if ((int64_t)t * kTeamBlock >= cp) {
        v = t;
        break;
      }
    const int64_t chunk = (int64_t)v * kTeamBlock;
    const int64_t wpc = (cp + chunk - 1) / chunk;
    const int64_t team = d.D * wpc;
    const int64_t cus = current_num_cus() * kTeamPerCu < kTeamMaxWorkgroups
                            ? current_num_cus() * kTeamPerCu
                            : kTeamMaxWorkgroups;
    const bool apart = !(ob < gb + nbytes && gb < ob + nbytes) && !(ob < xb + nbytes && xb < ob + nbytes);
    // (channels of at most 1024 packs -- one or two packs a lane -- move too little between
    // two exchanges: bf16 [2, 2048, 64, 64] in 32 groups, 8 rounds of 8 KB a workgroup and
    // tensor, 56.6 us against 35.0 us for the two launches)
    if (apart && v >= 4 && team >= 2 && team <= cus && 2 * cp >= wpc * chunk) {
      int64_t teams = cus / team;
      if (teams > d.rows) teams = d.rows;
      a.team = (int)team;
      a.team_wpc = (int)wpc;
      a.team_v = v;
      a.team_grid = teams * team;
      a.team_slot = team_slot_for_call(s, &a.team_id);
      a.team_wait_ticks = g_team_wait_ticks.load(std::memory_order_relaxed);
    }
  }
  if (xd == ROWNORM_F32) return launch_group_norm_bwd<float, float>(plan, a, s);
  if (xd == ROWNORM_F16)
    return wd == ROWNORM_F32 ? launch_group_norm_bwd<f16, float>(plan, a, s)
                             : launch_group_norm_bwd<f16, f16>(plan, a, s);
  return wd == ROWNORM_F32 ? launch_group_norm_bwd<bf16, float>(plan, a, s)
                           : launch_group_norm_bwd<bf16, bf16>(plan, a, s);
}

int mi355x_group_norm_plan(int backward, int64_t N, int64_t C, int64_t HxW, int64_t groups,
                           rownorm_dtype x_dtype, rownorm_plan* out) {
  if (!out) return ROWNORM_ERR_NULL;
  if (esize_of((int)x_dtype) == 0) return ROWNORM_ERR_DTYPE;
  GroupDims d;
  if (int e = group_dims(N, C, HxW, groups, &d)) return e;
  Plan plan;
  if (int e = group_plan(backward ? OC_GROUP_BWD : OC_GROUP_FWD,
                         backward ? ROWNORM_OP_GROUP_NORM_BWD : ROWNORM_OP_GROUP_NORM_FWD, d, HxW,
                         esize_of((int)x_dtype), &plan))
    return e;
  out->resident = plan.resident ? 1 : 0;
  out->lanes_per_row = plan.G;
  out->packs_per_lane = plan.V;
  out->block_threads = plan.block;
  out->rows_per_block = plan.rpb;
  out->reserved = plan.fast ? gn_mode(d.L, HxW, d.D, 16 / esize_of((int)x_dtype)) : kGnGeneral;
  out->grid_blocks = plan.grid;
  // (forward slabs beyond the registers whose channels are whole packs: the team launch)
  if (!backward && plan.team > 0 && HxW % (16 / esize_of((int)x_dtype)) == 0)
    out->grid_blocks = plan.team_grid;
  out->partial_rows = backward ? N : 0;
  return 0;
}

int mi355x_softmax_strided_fwd(const void* x, void* y, int64_t outer, int64_t dim_size,
                               int64_t inner, rownorm_dtype in_dtype, rownorm_dtype out_dtype,
                               int mode, void* stream) {
  const int id = (int)in_dtype, od = (int)out_dtype;
  int flags = 0;
  if (esize_of(id) == 0 || esize_of(od) == 0) return ROWNORM_ERR_DTYPE;
  if (!(od == id || (id == ROWNORM_F16 && od == ROWNORM_F32))) return ROWNORM_ERR_DTYPE;
  if (int e = strided_shape_check(outer, dim_size, inner)) return e;
  if (int e = softmax_mode_flags(mode, true, &flags)) return e;
  if (outer == 0 || dim_size == 0 || inner == 0) return 0;
  if (inner == 1)  // the reduced dimension is innermost after all
    return softmax_fwd(x, nullptr, y, outer, dim_size, MaskRows{}, id, od, flags, stream);
  if (!x || !y) return ROWNORM_ERR_NULL;
  StridedPlan plan;
  if (int e = make_strided_plan(false, outer, dim_size, inner, esize_of(id), current_num_cus(),
                                g_override[ROWNORM_OP_SOFTMAX_STRIDED_FWD], &plan))
    return e;
  SoftmaxStridedFwdArgs a{x, y, outer, (int)dim_size, (int)inner, flags};
  hipStream_t s = (hipStream_t)stream;
  if (id == ROWNORM_F32) return launch_softmax_strided_fwd<float, float>(plan, a, s);
  if (id == ROWNORM_BF16) return launch_softmax_strided_fwd<bf16, bf16>(plan, a, s);
  return od == ROWNORM_F32 ? launch_softmax_strided_fwd<f16, float>(plan, a, s)
                           : launch_softmax_strided_fwd<f16, f16>(plan, a, s);
}

int mi355x_softmax_strided_bwd(const void* grad, const void* y, void* gi, int64_t outer,
                               int64_t dim_size, int64_t inner, rownorm_dtype grad_dtype,
                               rownorm_dtype gi_dtype, int mode, void* stream) {
  const int gd = (int)grad_dtype, od = (int)gi_dtype;
  int flags = 0;
  if (esize_of(gd) == 0 || esize_of(od) == 0) return ROWNORM_ERR_DTYPE;
  if (!(od == gd || (gd == ROWNORM_F32 && od == ROWNORM_F16))) return ROWNORM_ERR_DTYPE;
  if (int e = strided_shape_check(outer, dim_size, inner)) return e;
  if (int e = softmax_mode_flags(mode, false, &flags)) return e;
  if (outer == 0 || dim_size == 0 || inner == 0) return 0;
  if (inner == 1)
    return softmax_bwd(grad, y, nullptr, gi, outer, dim_size, MaskRows{}, gd, od, flags, stream);
  if (!grad || !y || !gi) return ROWNORM_ERR_NULL;
  StridedPlan plan;
  if (int e = make_strided_plan(true, outer, dim_size, inner, esize_of(gd), current_num_cus(),
                                g_override[ROWNORM_OP_SOFTMAX_STRIDED_BWD], &plan))
    return e;
  SoftmaxStridedBwdArgs a{grad, y, gi, outer, (int)dim_size, (int)inner, flags};
  hipStream_t s = (hipStream_t)stream;
  if (gd == ROWNORM_BF16) return launch_softmax_strided_bwd<bf16, bf16>(plan, a, s);
  if (gd == ROWNORM_F16) return launch_softmax_strided_bwd<f16, f16>(plan, a, s);
  return od == ROWNORM_F16 ? launch_softmax_strided_bwd<float, f16>(plan, a, s)
                           : launch_softmax_strided_bwd<float, float>(plan, a, s);
}

int mi355x_softmax_strided_plan(int backward, int64_t outer, int64_t dim_size, int64_t inner,
                                rownorm_dtype dtype, rownorm_plan* out) {
  if (!out) return ROWNORM_ERR_NULL;
  if (esize_of((int)dtype) == 0) return ROWNORM_ERR_DTYPE;
  if (int e = strided_shape_check(outer, dim_size, inner)) return e;
  StridedPlan plan;
  const int op = backward ? ROWNORM_OP_SOFTMAX_STRIDED_BWD : ROWNORM_OP_SOFTMAX_STRIDED_FWD;
  if (int e = make_strided_plan(backward != 0, outer, dim_size, inner, esize_of((int)dtype),
                                current_num_cus(), g_override[op], &plan))
    return e;
  out->resident = plan.resident ? 1 : 0;
  out->lanes_per_row = 1 << plan.tx_log2;
  out->packs_per_lane = plan.V;
  out->block_threads = plan.block;
  out->rows_per_block = 1 << plan.ty_log2;
  out->reserved = plan.chunks > 1 ? plan.chunks : 0;
  out->grid_blocks = plan.grid;
  out->partial_rows = 0;
  return 0;
}

int mi355x_rownorm_plan_at(rownorm_op op, int64_t M, int64_t N, rownorm_dtype x_dtype,
                           rownorm_dtype w_dtype, int off_line, rownorm_plan* out) {
  if ((int)op < 0 || (int)op > ROWNORM_OP_SOFTMAX_BWD) return ROWNORM_ERR_SHAPE;
  if (!out) return ROWNORM_ERR_NULL;
  if (esize_of((int)x_dtype) == 0) return ROWNORM_ERR_DTYPE;
  if (int e = shape_check(M, N)) return e;
  Plan plan;
  const OpClass oc = class_of((int)op);
  const bool layer_norm = op == ROWNORM_OP_LAYER_NORM_FWD || op == ROWNORM_OP_LAYER_NORM_BWD;
  // the norm backward does not look at its pointers
  const bool off = off_line != 0 && oc != OC_NORM_BWD;
  if (int e = make_plan(oc, M, N, esize_of((int)x_dtype), current_num_cus(), g_override[(int)op],
                        oc == OC_NORM_BWD, &plan, false, layer_norm,
                        esize_of((int)w_dtype) > esize_of((int)x_dtype), off))
    return e;
  out->resident = plan.resident ? 1 : 0;
  out->lanes_per_row = plan.G;
  out->packs_per_lane = plan.V;
  out->block_threads = plan.block;
  out->rows_per_block = plan.rpb;
  // (a forward row held by a team of workgroups: the team and its grid)
  out->reserved = plan.team > 0 ? plan.team : (plan.split > 1 ? plan.split : 0);
  out->grid_blocks = plan.team > 0 ? plan.team_grid : plan.grid;
  out->partial_rows = (int64_t)bwd_partial_rows(plan);
  // (groups of rows held by teams: the workgroup, the packs of a row a lane holds, the rows)
  if (plan.team > 0 && (op == ROWNORM_OP_LAYER_NORM_BWD || op == ROWNORM_OP_RMS_NORM_BWD)) {
    out->lanes_per_row = kTeamBlock;
    out->block_threads = kTeamBlock;
    out->packs_per_lane = plan.team_v;
    out->rows_per_block = kTeamBwdRows;
  }
  if (plan.team > 0 && plan.team_r > 0) {
    out->lanes_per_row = kTeamBlock;
    out->block_threads = kTeamBlock;
    out->packs_per_lane = plan.team_v;
    out->rows_per_block = plan.team_r;
  }
  return 0;
}

int mi355x_rownorm_plan(rownorm_op op, int64_t M, int64_t N, rownorm_dtype x_dtype,
                        rownorm_dtype w_dtype, rownorm_plan* out) {
  return mi355x_rownorm_plan_at(op, M, N, x_dtype, w_dtype, 0, out);
}

int mi355x_rownorm_set_override(rownorm_op op, int lanes_per_row, int packs_per_lane,
                                int block_threads, int blocks_per_cu) {
  if ((int)op < 0 || (int)op >= ROWNORM_OP_COUNT) return ROWNORM_ERR_SHAPE;
  if (lanes_per_row < -1 || lanes_per_row > 0x7fff || packs_per_lane < 0 ||
      packs_per_lane > 0xffff || block_threads < 0 || block_threads > 0xffff ||
      blocks_per_cu < 0 || blocks_per_cu > 0xffff)
    return ROWNORM_ERR_OVERRIDE;
  Override o;
  o.G = lanes_per_row;
  o.V = packs_per_lane;
  o.block = block_threads;
  o.bpc = blocks_per_cu;
  g_override_bits[(int)op].store(pack_override(o), std::memory_order_relaxed);
  return 0;
}

int mi355x_rownorm_set_team_wait_us(unsigned int microseconds) {
  g_team_wait_ticks.store(microseconds == 0xffffffffu ? 100000000ull
                                                      : (unsigned long long)microseconds * 100ull,
                          std::memory_order_relaxed);
  return 0;
}

}  // extern "C"
