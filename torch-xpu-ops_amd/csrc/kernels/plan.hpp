// Host-side choice of the launch layout for one call (no HIP types in here).
//
// Stands in for the reference's work-split heuristics: NormConfig
// (src/ATen/native/xpu/sycl/Norm.h:225-370), layer_norm_wg_size_select
// (LayerNormKernels.cpp:588-616) and get_wgroup_size (SoftMaxKernels.cpp:
// 139-182).  Those are written around Intel EU counts and SIMD32 sub-groups;
// here the split is a small table over the row size for 256 compute units of
// 64-wide wavefronts.
//
// The rule.  A row of N elements is ceil(N / E) 16-byte packs (E = 4 for fp32,
// 8 for 16-bit types).  G lanes share a row and each holds V packs:
//   G = smallest power of two in [8, 1024] with G * V_pref >= packs,
//   V = smallest power of two with G * V >= packs.
// If V exceeds the per-op register budget V_max the multi-pass streaming
// kernel is used instead.  Rows whose length is a whole number of packs take
// the branch-free "fast" kernels; ragged rows (N % E != 0) take the general
// ones, which exist for V = V_pref only (and three packs for 16-bit softmax and
// the 16-bit norms).  Measured exceptions for rows that
// leave many of those lanes idle (hidden sizes that are not powers of two) or
// that would take 1024 lanes: norm_layout() and the softmax / GroupNorm rules
// in make_plan() pick three or five packs a lane, or fewer lanes.  Workgroup
// size and grid size per op class are set by block_threads() and default_bpc()
// below.
#pragma once
#include <stdint.h>

namespace rownorm {

enum OpClass {
  OC_NORM_FWD = 0,
  OC_NORM_BWD = 1,
  OC_SOFTMAX_FWD = 2,
  OC_SOFTMAX_BWD = 3,
  OC_GROUP_FWD = 4,  // GroupNorm: rows are (sample, group) slabs, no per-column registers
  OC_GROUP_BWD = 5
};

struct Override {
  // 0 = automatic; G = -1 = force the streaming kernel, and then V = 1 keeps every
  // row on one workgroup, V > 1 splits every row over V workgroups (norm ops), V = 0 with
  // block = 1 sends a norm backward of whole packs to teams of workgroups however few
  // rounds they make
  int G = 0, V = 0, block = 0, bpc = 0;
};

struct Plan {
  bool resident = true;
  bool fast = true;  // N % E == 0: branch-free row access
  int G = 0, V = 0, block = 0, rpb = 0;
  int64_t grid = 0;
  int64_t partial_rows = 0;
  // Split-row path of the norm ops (few rows, each far too long for registers):
  // a row is cut into `split` chunks of `chunk_packs` packs, one workgroup each;
  // 0 or 1 = one workgroup per row.
  int split = 0;
  int64_t chunk_packs = 0;
  // softmax backward of rows beyond the registers of two tensors: grad alone fits
  // them (the log_softmax backward then keeps grad resident and streams y)
  bool grad_resident = false;
  // a layout was asked for by override: kernels chosen by other means than the
  // layout (softmax of short ragged rows through LDS) stand back
  bool forced = false;
  // norm forward of rows beyond one workgroup's registers held by a team of
  // workgroups (norm_fwd_team_kernel): workgroups a row, packs a lane the kernel is
  // compiled for, packs a workgroup, workgroups launched; team == 0: not planned
  int team = 0, team_v = 0;
  int64_t team_chunk_packs = 0, team_grid = 0;
  // norm backward of such rows held R = team_v rows at a time by teams of workgroups
  // (norm_bwd_team_kernel): the same fields, one stride of packs a workgroup, and the
  // partial rows of column sums that launch leaves (one a team; partial_rows is what
  // the kernels behind it would use)
  int64_t team_partial_rows = 0;
  // norm forward of such rows with three rows in flight a workgroup, team_v packs of a row
  // a lane and the weights held (norm_fwd_rows_team_kernel): 1; 0: norm_fwd_team_kernel
  int team_r = 0;
  // norm backward / forward on an exact layout (norm_bwd_exact_kernel,
  // norm_fwd_exact_kernel): row blocks a lane keeps in flight, itself included (the
  // forward: 1); GroupNorm on an exact layout (gn_*_exact_kernel): 1; 0 = the
  // general resident kernel
  int exact_depth = 0;
  // ragged 16-bit norm rows addressed through the 16-byte aligned window that holds
  // each row (norm_row_window()): G * V holds the packs of that window, and a
  // workgroup that walks several row blocks strides by a multiple of 8 rows
  bool window = false;
};

// norm_fwd_team_kernel: threads a workgroup, packs a lane at most, workgroups of
// the grid at most (one a compute unit), slots of bookkeeping memory.
constexpr int kTeamBlock = 512;
constexpr int kTeamPerCu = 2;  // workgroups of a team launch a compute unit holds
constexpr int kTeamMaxV = 16;
constexpr int kTeamGroup = 2;  // packs whose weights are requested together
constexpr int kTeamMaxWorkgroups = 512;
constexpr int kTeamSlots = 16;
constexpr int kTeamMinTeams = 8;
// norm_bwd_team_kernel: rows a team holds at a time, packs of a row a lane holds of each
// tensor, workgroups a compute unit
constexpr int kTeamBwdRows = 4;
constexpr int kTeamBwdPacks = 2;
constexpr int kTeamBwdPerCu = 1;
// norm_fwd_rows_team_kernel: packs of a row a lane, and the rounds from which it is taken
constexpr int kTeamFwdLongPacks = 10;
constexpr int kTeamFwdMinRounds = 16;
// One call's bookkeeping memory (see the kernel).
struct TeamEntry {
  // the two-number exchange: (call id << 32) | (round + 1) once s1, s2 are in place, 0 while
  // they change; a workgroup's partial sums (float64 bit patterns)
  unsigned long long tag;
  unsigned long long s1, s2;
  // the exchanges of self-validating words {32 bits of payload, tag}: see device/team.hpp
  // (128 bytes an entry: neighbours' polls go to other memory channels)
  unsigned long long pad[13];
};
struct TeamSlot {
  // [round parity][workgroup]; norm_bwd_team_kernel, which publishes a round before it
  // gathers the one before, goes round all four
  TeamEntry entry[4][kTeamMaxWorkgroups];
  unsigned int gave_up;                    // id of a call one of whose waits ran out (a hint)
  unsigned int pad[3];
};

// softmax_fwd_team_kernel / softmax_bwd_team_kernel: rows of at least this many packs (64 KiB),
// and the packs a lane the backward holds of each of its two tensors at most.
constexpr int64_t kSoftmaxTeamMinPacks = 4096;
constexpr int kSoftmaxBwdTeamMaxV = 8;

constexpr int kMinG = 8;
constexpr int kMaxG = 1024;
constexpr int kMaxV = 16;
// The 16-bit softmax forward alone goes to 20 packs a lane (163840-element rows:
// the 151936 / 152064-entry vocabularies).
constexpr int kSoftmaxFwdMaxV16 = 20;
// Packs of grad a lane of the grad-resident log_softmax backward holds at most.
constexpr int kGradResidentMaxV = 20;
constexpr int max_v_of(OpClass oc, int esize) {
  return oc == OC_SOFTMAX_FWD && esize == 2 ? kSoftmaxFwdMaxV16 : kMaxV;
}
constexpr int kStreamBlock = 1024;
// Split-row path: a chunk is a whole number of workgroup strides and at least
// four of them (32768 16-bit elements); a row is cut into at most 1024 chunks.
constexpr int kSplitMinStrides = 4;
constexpr int kSplitMaxChunks = 1024;

// Preferred packs per lane: what the G ladder aims for.
// Measured on MI355X: 16 elements a lane (two 16-bit packs, four fp32 packs)
// keeps the register count low enough for 8 wavefronts per SIMD, which beats
// fewer, fatter lanes on every op of the family.
constexpr int v_pref(OpClass, int esize) { return esize == 4 ? 4 : 2; }

// Ragged 16-bit rows of the norm forward (every row at another 2-byte alignment,
// where a 128-bit access costs about twice an aligned one) on 256 lanes or more are
// addressed through the 16-byte aligned window that holds the row: it starts up to
// 7 elements before the row and can hold one pack more than the row.  Every whole
// pack of the window is an aligned access, the two end packs are trimmed (loads)
// or written element by element (stores), and gamma / beta are held shifted by the
// window's head: loaded once per workgroup when all its rows have the same head,
// i.e. when it strides by a multiple of 8 rows, which make_plan() sees to (and
// again per row otherwise).  fp16, 8192 rows that start 2 elements into their
// buffers: N = 4097 LayerNorm 43.6 -> 34.6 us, RMSNorm 31.2 -> 29.9 us; 8193: 68.8 ->
// 61.0 and 58.9 -> 51.1 us.  Shorter rows lose (the two end packs weigh more: N =
// 2049 LayerNorm 20.0 -> 20.9 us, RMSNorm 15.3 -> 17.3 us) and keep the row-start
// addressing; so does the backward, which measured no gain (N = 4097 LayerNorm 68.6
// -> 68.1 us) or a loss (RMSNorm 53.8 -> 71.6 us: 132 registers against 127, one
// workgroup a compute unit instead of two).
constexpr bool norm_row_window(int esize, int G, bool fast) {
  return !fast && esize == 2 && G >= 256;
}

// The resident norm forward keeps gamma / beta of a lane's columns in registers
// across its rows while they fit; at 1024 lanes, rows of more packs a lane than
// the table below leave the weights in memory, load each pack of them (from L2)
// where the output needs it, and hold only the row.  esize / wsize: bytes of a
// row / weight element.  Measured, bf16 rows, against the multi-pass kernel that
// served rows beyond 4 packs a lane before (2048 rows): N = 40960 LayerNorm 84 ->
// 65 us (fp32 weights 90 -> 72), RMSNorm 66 -> 59; 65536: 109 -> 101 and 104 ->
// 95; 1024 rows of 131072: 114 -> 105 and 114 -> 98.  Held against looked up, where
// both fit the registers (8192 rows of 40960 / 4096 of 49152 / 8192 of 65536):
// LayerNorm bf16 weights 226 / 143 us against 244 / 153; RMSNorm bf16 weights 240 /
// 147 / 373 against 227 / 144 / 384 (5 and 6 packs held leave one workgroup a
// compute unit where the lookup keeps two); RMSNorm fp32 weights 222 / 136 / 400
// against 236 / 145 / 395.  Up to 4 packs the held weights win by 5-20 %.  The fp32
// LayerNorm with its weights held spilled from 5 packs a lane (N = 20480..32768:
// 209..229 -> 62..104 us); the fp32 RMSNorm holds 8 packs and is 3 % faster so.
constexpr int kNormFwdHoldMaxV = 4;
// With the residual add fused in (a second row in flight a lane) only the lookup
// fits beyond 4 packs, and rows up to norm_fwd_add_max_v() packs a lane.
constexpr bool norm_fwd_holds_weights(int esize, int wsize, int G, int V, bool fast, bool rms,
                                      bool add) {
  if (!fast || G != 1024 || V <= kNormFwdHoldMaxV) return true;
  if (add) return false;
  if (esize == 4) return rms && V <= 8;
  if (wsize == 2) return rms ? V == 8 : V <= 6;
  return rms && V <= 6;
}

constexpr int norm_fwd_add_max_v(int esize, bool rms) { return esize == 4 && !rms ? 10 : 12; }

// Largest packs per lane the register file holds for a G-lane row group.
// G = 1024 means 16 wavefronts per workgroup, i.e. at most 128 VGPRs a lane.
constexpr int v_max(OpClass oc, int esize, int G) {
  int v = 1;
  switch (oc) {
    // (at 1024 lanes without the weights: 16 packs, a 131072-element 16-bit row or
    // a 65536-element fp32 row)
    case OC_NORM_FWD:
      if (G >= 1024) return 16;
      v = esize == 4 ? 16 : 8;
      break;
    // (16-bit rows at 1024 lanes: 4 packs with the dgamma sums in LDS, see
    // norm_bwd_sums_in_lds())
    case OC_NORM_BWD:
      if (G >= 1024 && esize == 2) return 4;
      if (G == 512 && esize == 2) return 5;  // (5: norm_bwd_half_lanes_five())
      v = esize == 4 ? 8 : 4;
      break;
    // the forward keeps long rows in storage format: 16 packs a lane at any
    // G (a 131072-element 16-bit row, a 65536-element fp32 row)
    case OC_SOFTMAX_FWD: return G >= 1024 ? max_v_of(oc, esize) : 16;
    // (16-bit rows at 1024 lanes: 8 packs of each tensor, kept in storage format)
    case OC_SOFTMAX_BWD:
      if (G >= 1024 && esize == 2) return 8;
      v = esize == 4 ? 16 : 8;
      break;
    // GroupNorm lanes hold the row (and dY) only, no weights or column sums, so
    // 16-bit rows keep 8 packs a lane at 1024 lanes (128 VGPRs) and 10 at 512
    // lanes (two workgroups a compute unit); the fp32 forward holds 11 at 1024
    // lanes without spilling, the fp32 backward 4
    case OC_GROUP_FWD: return esize == 4 ? (G >= 1024 ? 11 : 16) : (G == 512 ? 10 : 8);
    case OC_GROUP_BWD: return esize == 4 ? (G >= 1024 ? 4 : 8) : 8;
  }
  if (G >= 1024 && v > 1) v /= 2;
  return v;
}

// Threads per workgroup for a G-lane row group (measured choices):
//   norm forward    256 (BLOCK/G rows per workgroup), G itself above that;
//   norm backward   512 at least: two or more row slots share one partial row
//                   of the dgamma/dbeta reduction;
//   softmax         512 at least;
//   GroupNorm       256 in both directions: its backward keeps no column sums across
//                   rows (the channel sums of a row leave with the row), and with 256
//                   threads bf16 [256, 1024, 14, 14] in 32 groups went 72.0 -> 62.7 us
//                   (dX kernel alone), [256, 2048, 7, 7] 38.8 -> 35.8 us, [64, 1280, 8, 8]
//                   unchanged, [64, 1280, 16, 16] 23.7 -> 24.3 us.
constexpr int block_threads(OpClass oc, int G) {
  const int floor_threads =
      (oc == OC_NORM_FWD || oc == OC_GROUP_FWD || oc == OC_GROUP_BWD) ? 256 : 512;
  return G <= floor_threads ? floor_threads : G;
}

// Whether the resident norm backward requests the rows of its next iteration
// ahead of the current one's arithmetic.  That costs V * 8 registers a lane for
// 16-bit rows.  The two-pack layouts sit just under 128 registers, which keeps
// two 512-thread workgroups on a compute unit, and lose more to a lost
// workgroup than they gain (bf16 [16384, 4096] LayerNorm 78 -> 85 us; with the
// dgamma/dbeta sums moved to LDS to make room, read-add-write 128 bits at a
// time, 78 -> 82 us, and with LDS float atomics ten times that); from three packs
// a lane the kernel holds one workgroup a compute unit anyway and has the
// registers to spare (N = 10240: LayerNorm 208 -> 185 us, RMSNorm 189 -> 176 us;
// with one workgroup a compute unit in the grid as well, see make_plan(), 173
// and 169 us).  The two-pack LayerNorm, whose two sets of column sums make it
// the slower one, gains a little from the prefetch on one workgroup a compute
// unit up to 256 lanes (N = 2048: 44.6 -> 43.3 us, 4096: 78 -> 75 us) and loses a
// little on 512 (N = 7168: 128 -> 130 us, 8192: 142 -> 144 us).
constexpr bool norm_bwd_prefetches(int esize, int G, int V, bool fast, bool rms) {
  if (G >= 1024) return false;  // (3 and 4 packs at 1024 lanes: it spills, 104 -> 172 us)
  return fast && esize == 2 && (V >= 3 || (V == 2 && !rms && G <= 256));
}

// 16-bit backward rows of 16392..32768 elements (hidden sizes 18432, 20480): three
// or four packs a lane on 1024 lanes.  The column sums of such a lane would take
// 48-64 registers beside the row and dY, so the dgamma sums live in LDS (96 / 128
// KB: every lane adds to its own 16-byte slots), the dbeta sums stay in registers
// and gamma stays in memory (L2).  Measured at 4096 rows against the multi-pass
// kernels (two passes over X and dY), bf16: N = 18432 RMSNorm 127 -> 104 us,
// LayerNorm 133 -> 111 us (fp32 weights 147 -> 126 us); 24576: 162 -> 135, 166 ->
// 143, 180 -> 151 us; 32768 RMSNorm 231 -> 175 us.  The LayerNorm with four packs
// spills 29-45 registers and loses (237 -> 302 us): it keeps the multi-pass kernels.
constexpr bool norm_bwd_sums_in_lds(int esize, int G, int V, bool fast) {
  return fast && esize == 2 && G == 1024 && V >= 3;
}
// One case goes through the registers instead: the RMSNorm with 16-bit weights and
// rows of 2049..2560 packs (hidden 18432, 20480) fits 512 lanes x 5 packs with its
// next row on the way in 251 registers, one 512-thread workgroup a compute unit
// (bf16 [16384, 18432] 345 -> 315 us, 72 %; [8192, 20480] 194 -> 176 us).  The
// LayerNorm, fp32 weights and the fused residual gradient spill there (LayerNorm
// 199 -> 351 us) and stay with the LDS sums; so do 6 packs (24576).
constexpr bool norm_bwd_half_lanes_five(int esize, int wsize, int G, int V, bool rms, bool add) {
  return esize == 2 && wsize == 2 && G == 512 && V == 5 && rms && !add;
}
// Exact layouts of the 16-bit norm backward (norm_bwd_exact_kernel): a row of
// `packs` = V * G packs on G lanes, G a whole number of wavefronts.  The table is
// what measured faster than the general resident kernel on MI355X (see the kernel):
// lanes, packs a lane, workgroup threads, row blocks in flight (1 = no prefetch),
// and which calls take it -- LayerNorm / RMSNorm, weights in the row dtype / in
// float32 beside 16-bit rows, with the residual gradient fused in or not.  Two packs
// a lane serve hidden sizes up to 16384; three and four packs a lane keep rows of
// 9216, 18432, 20480 and 24576 elements in registers where the general kernel needs
// its dgamma sums in LDS (bf16 rows x 8192, LayerNorm 18432: 199 -> 165 us, with fp32
// weights 231 -> 166 us; 24576: 258 -> 222 us; RMSNorm with fp32 weights 18432 185 ->
// 158 us, 20480 206 -> 181 us, 24576 231 -> 212 us).
constexpr unsigned kExactLN = 1, kExactLNWide = 2, kExactRMS = 4, kExactRMSWide = 8,
                   kExactAdd = 16;  // (kExactAdd: also with the fused residual gradient)
constexpr unsigned kExactAll = kExactLN | kExactLNWide | kExactRMS | kExactRMSWide;
struct NormBwdExactLayout {
  int G, V, block, depth;
  unsigned calls;
};
constexpr NormBwdExactLayout kNormBwdExact[] = {
    {128, 2, 512, 2, kExactAll | kExactAdd},
    // (the first entry that serves a call is taken: one row slot a workgroup where that
    // measured ahead -- bf16 rows x 16384, LayerNorm 4096 69.4 -> 68.8 us, 5120 88.7 ->
    // 86.5 us, RMSNorm 5120 86.0 -> 83.2 us, 6144 on 384 x 2 instead of 256 x 3 LayerNorm
    // 105.9 -> 102.1 us (fp32 weights 107.3 -> 102.6), RMSNorm 101.9 -> 99.7 us)
    {256, 2, 256, 3, kExactLN | kExactLNWide},
    {256, 2, 512, 3, kExactAll | kExactAdd},
    {320, 2, 320, 3, kExactLN | kExactLNWide},
    {320, 2, 320, 2, kExactRMS | kExactRMSWide},
    {320, 2, 640, 2, kExactAll | kExactAdd},
    {384, 2, 384, 2, kExactAll},
    {448, 2, 448, 2, kExactAll | kExactAdd},
    {512, 2, 512, 3, kExactAll | kExactAdd},
    // (at 896 and 1024 lanes the RMSNorm's general kernel already runs this layout as fast)
    {896, 2, 896, 1, kExactLN | kExactLNWide | kExactAdd},
    {1024, 2, 1024, 1, kExactLN | kExactLNWide | kExactAdd},
    {384, 3, 384, 2, kExactAll},
    {768, 3, 768, 1, kExactLN | kExactLNWide | kExactRMSWide},
    {640, 4, 640, 1, kExactRMSWide},
    {1024, 3, 1024, 1, kExactAll}};
constexpr int kNormBwdExactCount = (int)(sizeof(kNormBwdExact) / sizeof(kNormBwdExact[0]));
constexpr bool norm_bwd_exact_serves(const NormBwdExactLayout& l, bool layer_norm,
                                     bool wide_weights, bool fused_add) {
  const unsigned want = layer_norm ? (wide_weights ? kExactLNWide : kExactLN)
                                   : (wide_weights ? kExactRMSWide : kExactRMS);
  return (l.calls & want) != 0 && (!fused_add || (l.calls & kExactAdd) != 0);
}
// Index into kNormBwdExact of the layout that serves such a call, or -1.
constexpr int norm_bwd_exact_index(int esize, int64_t packs, int64_t M, bool layer_norm,
                                   bool wide_weights, bool fused_add) {
  if (esize != 2) return -1;
  for (int i = 0; i < kNormBwdExactCount; ++i) {
    const NormBwdExactLayout& l = kNormBwdExact[i];
    if (packs == (int64_t)l.V * l.G && norm_bwd_exact_serves(l, layer_norm, wide_weights, fused_add) &&
        M % (l.block / l.G) == 0)
      return i;
  }
  return -1;
}
// Exact two-pack layouts of the 16-bit norm forward (norm_fwd_exact_kernel): lanes,
// workgroup threads, resident workgroups a compute unit.  Hidden 4096 and 5120, where
// it measured 2-5 % ahead of the general resident kernel; not 8192.
struct NormFwdExactLayout {
  int G, block, bpc;
};
constexpr NormFwdExactLayout kNormFwdExact[] = {{256, 512, 2}, {320, 320, 3}};
constexpr int kNormFwdExactCount = (int)(sizeof(kNormFwdExact) / sizeof(kNormFwdExact[0]));
// (up to 128 row blocks a workgroup: at 262144 rows of 4096 the resident grid runs
// at 68 % where the general kernel's grid, which grows with the rows, reaches 75 %)
constexpr int kNormFwdExactMaxIters = 128;
constexpr int norm_fwd_exact_index(int esize, int64_t packs, int64_t M, int num_cus) {
  if (esize != 2) return -1;
  for (int i = 0; i < kNormFwdExactCount; ++i) {
    const int rpb = kNormFwdExact[i].block / kNormFwdExact[i].G;
    if (packs == 2 * (int64_t)kNormFwdExact[i].G && M % rpb == 0 &&
        M / rpb <= (int64_t)num_cus * kNormFwdExact[i].bpc * kNormFwdExactMaxIters)
      return i;
  }
  return -1;
}
// Exact layouts of the 16-bit GroupNorm kernels (gn_fwd_exact_kernel,
// gn_bwd_exact_kernel): one row a workgroup of G lanes with V packs each, for
// rows of exactly G * V packs whose channels are whole runs of 64 packs (the
// 64x64 and 32x32 maps of a diffusion UNet with 32 groups: 10, 20, 30, 40 and 60
// channels a group at 32x32, 10 at 64x64).  Workgroups a compute unit of the
// forward and of the backward grid; 0 = the general resident kernel is faster
// (measured on one MI355X, bf16, 2048 rows; general -> exact, us:
//   1280 packs  forward 14.2 -> 15.0 (kept general)   backward 26.4 -> 22.2
//   2560 packs  forward 29.9 -> 29.3                  backward 49.3 -> 43.0
//   3840 packs  forward 46.6 -> 43.8                  backward 79.4 -> 67.9
//   5120 packs  forward 61.6 -> 58.6                  backward 96.2 -> 84.9 + 3.5
//               (one row a workgroup: 2048 workgroups; a grid of 512 is 2 % behind)
//   7680 packs  forward 94.7 -> 90.2                  backward 140.6 -> 128.0).
struct GroupExactLayout {
  int G, V, bpc_fwd, bpc_bwd;
};
constexpr GroupExactLayout kGroupExact[] = {
    {256, 5, 0, 8}, {512, 5, 3, 2}, {768, 5, 2, 1}, {512, 10, 8, 8}, {960, 8, 1, 1}};
constexpr int kGroupExactCount = (int)(sizeof(kGroupExact) / sizeof(kGroupExact[0]));
constexpr int kGroupExactMaxD = 64;  // channels a group: one lane of a wavefront each
constexpr int group_exact_index(bool backward, int esize, int64_t rows, int64_t L, int64_t HxW,
                                int64_t D) {
  const int E = 8;
  if (esize != 2 || L % E != 0 || HxW % (64 * E) != 0 || D > kGroupExactMaxD ||
      rows > ((int64_t)1 << 31))
    return -1;
  for (int i = 0; i < kGroupExactCount; ++i) {
    const GroupExactLayout& l = kGroupExact[i];
    if (L / E == (int64_t)l.G * l.V && (backward ? l.bpc_bwd : l.bpc_fwd) > 0) return i;
  }
  return -1;
}
// (a 512 x 5 instance exists for that case only)
constexpr bool norm_bwd_instance_ok(int esize, int wsize, int G, int V, bool rms, bool add) {
  return !(esize == 2 && G == 512 && V == 5) || norm_bwd_half_lanes_five(esize, wsize, G, V, rms, add);
}
constexpr bool norm_bwd_lds_layout(int esize, int64_t v_exact, bool layer_norm) {
  return esize == 2 && (v_exact == 3 || (v_exact == 4 && !layer_norm));
}

// Workgroup sizes a G-lane variant is compiled for.
constexpr bool block_built(OpClass oc, int G, int block) {
  if (block < G || block < 256 || block > 1024 || (block & (block - 1))) return false;
  return block == block_threads(oc, G);
}

// Workgroups per compute unit of the grid-stride launch.  The norm kernels keep
// gamma/beta (and the backward column sums) in registers across the rows of a
// workgroup.  Forward: four times as many workgroups as fit on the machine at
// once, so that they drift out of phase (a grid that is exactly resident runs
// its load and store phases in lockstep and loses 5-10% bandwidth) while each
// still amortizes its weight loads over several rows (make_plan() grows this
// grid with the row count).  Backward: every
// workgroup emits one partial row of the dgamma/dbeta reduction, so the grid
// is just what is resident at 1024 threads per CU.  Softmax has no per-column
// state: one workgroup per row block.
constexpr int default_bpc(OpClass oc, int block) {
  if (oc == OC_NORM_FWD) return 4 * (2048 / block);
  if (oc == OC_NORM_BWD) return 1024 / block;
  return 1 << 20;
}

// Which (G, V) kernels exist in the library.  Kept in one place so the
// dispatcher, the planner and the forced-variant check agree.
constexpr bool is_group_class(OpClass oc) { return oc == OC_GROUP_FWD || oc == OC_GROUP_BWD; }

// Kinds of register-resident GroupNorm kernel (see groupnorm_kernels.hpp) and the
// rule that picks one for a shape; E = elements per 16-byte pack of the row dtype.
constexpr int kGnGeneral = 0, kGnUniform = 1, kGnStraddle = 2;
// Channels per group up to which the straddling kernels are taken (their LDS
// array for the parts of packs that belong to the next channel).
constexpr int kGnStraddleMaxD = 512;
constexpr int gn_mode(int64_t L, int64_t HxW, int64_t D, int E) {
  if (HxW % E == 0) return kGnUniform;
  if (L % E == 0 && HxW >= E && D <= kGnStraddleMaxD) return kGnStraddle;
  return kGnGeneral;
}

// GroupNorm rows that would spread over 1024 lanes (one workgroup a compute
// unit, whose load, reduce and store phases then run one after the other) take
// 512 lanes with twice the packs instead while two such workgroups fit a compute
// unit's registers (128 VGPRs a lane): up to 10 packs forward, 7 backward.
// Measured on [64, C, 64, 64] in 32 groups: bf16 forward 71 -> 62 us (C = 320),
// 57 -> 47 us (224); backward 76 -> 63 us (192), 88 -> 71 us (224); fp32
// backward 66 -> 59 us (96).  Eight packs backward spill and gain nothing.
constexpr int group_half_lanes_max_v(OpClass oc) { return oc == OC_GROUP_FWD ? 10 : 7; }

// Masked softmax rows are attention scores: the masked kernels exist up to 32
// elements a lane at 1024 lanes (rows of 32768 elements; the masked 16-bit
// backward, which keeps fp32 copies of both tensors, would spill beyond that
// anyway), and longer masked rows take the multi-pass kernels.
constexpr bool masked_softmax_built(int esize, int G, int V) {
  return !(G == 1024 && V * (16 / esize) > 32);
}

constexpr bool variant_built(OpClass oc, int esize, int G, int V, bool fast) {
  if (G < kMinG || G > kMaxG || (G & (G - 1)) || V < 1 || V > max_v_of(oc, esize)) return false;
  // GroupNorm rows take the packs they have, not the next power of two (a
  // 40960-element bf16 row is 1024 lanes x 5 packs, not x 8): 3 or 5 packs a
  // lane from one wavefront up, anything up to the budget at 1024 lanes
  if (V & (V - 1)) {
    // ragged 16-bit rows just above a power of two (softmax N = 4097: 514 packs of
    // the aligned window) take three packs on half the lanes as well
    if (!fast)
      return (oc == OC_SOFTMAX_FWD || oc == OC_SOFTMAX_BWD || oc == OC_NORM_FWD || oc == OC_NORM_BWD) && esize == 2 &&
             G >= 64 && V == 3 && !(oc == OC_NORM_BWD && G == kMaxG);
    if (V > v_max(oc, esize, G)) return false;
    // softmax rows that need all 1024 lanes (vocabulary-sized) likewise
    // (and the 16-bit forward takes three packs a lane where that fits better)
    if (oc == OC_SOFTMAX_FWD && esize == 2) return G == kMaxG || (G >= 64 && V == 3);
    if (oc == OC_SOFTMAX_FWD || oc == OC_SOFTMAX_BWD) return G == kMaxG;
    // LayerNorm / RMSNorm rows of hidden sizes such as 5120, 6144, 10240, 12288
    // (640, 768, 1280, 1536 16-bit packs): 3 packs a lane; 5 on 512 lanes for the
    // fp32 LayerNorm forward (see norm_layout())
    if (!is_group_class(oc)) {
      if (oc == OC_NORM_BWD && G == 512 && esize == 2 && V == 5) return true;
      // (16-bit forward rows of 2049..3072 packs: 5 or 6 packs on 512 lanes, see make_plan())
      if (oc == OC_NORM_FWD && G == 512 && esize == 2 && (V == 5 || V == 6)) return true;
      if (oc == OC_NORM_FWD && G == kMaxG && V > kNormFwdHoldMaxV)
        return V == 5 || V == 6 || V == 10 || V == 12;
      return G >= 64 && (V == 3 || (V == 5 && oc == OC_NORM_FWD && esize == 4 && G == 512));
    }
    // (and 6..10 packs on 512 lanes, which make_plan() prefers to 1024 lanes)
    return G == kMaxG || (G >= 64 && (V == 3 || V == 5)) ||
           (G == 512 && V <= group_half_lanes_max_v(oc));
  }
  if (V > v_max(oc, esize, G)) return false;
  // ragged rows: the general kernels exist for the preferred packs per lane only;
  // longer ragged rows take the multi-pass kernels (measured faster for softmax
  // at vocabulary sizes such as 50257 than a general kernel with more packs)
  if (!fast) return V == v_pref(oc, esize);
  if (G == kMinG) return V <= v_pref(oc, esize);
  // short rows take one pack a lane on up to one wavefront (see make_plan())
  if ((oc == OC_NORM_FWD || oc == OC_NORM_BWD || oc == OC_SOFTMAX_FWD || oc == OC_SOFTMAX_BWD) &&
      G <= 64 && V == 1)
    return true;
  if (is_group_class(oc) || G == kMaxG) return V >= v_pref(oc, esize);
  // below the lane maximum make_plan() takes the preferred packs a lane (more lanes
  // before more packs), with one measured exception: 16-bit norm rows of 1537..2048
  // packs on 512 lanes x 4.  Other layouts are never selected and are not compiled
  // (a third of the kernels otherwise).
  if ((oc == OC_NORM_FWD || oc == OC_NORM_BWD) && esize == 2 && G == 512 && V == 4) return true;
  return V == v_pref(oc, esize);
}

inline int pow2_ceil(int64_t v) {
  int p = 1;
  while (p < v) p <<= 1;
  return p;
}

// LayerNorm / RMSNorm rows that the power-of-two rule serves badly (measured on
// MI355X at 16384 rows; "slots" = lanes x preferred packs of that rule):
//  * a 16-bit row of 1025..2048 packs would take 1024 lanes, 16 wavefronts around
//    every reduction: 512 lanes with 3 or 4 packs each are faster in the forward
//    (LayerNorm 160 -> 116 us at N = 10240, RMSNorm 2-4 %) and in the LayerNorm
//    backward (250 -> 206 us); the RMSNorm backward gains only with 3 packs
//    (N = 12288: 222 -> 212 us) and keeps 1024 lanes beyond 1536 packs;
//  * a row that fills at most three quarters of the slots takes three packs on a
//    quarter of the slots' lanes instead: hidden sizes such as 1536, 3072, 6144,
//    12288 fit exactly, 2560, 5120, 10240 to 83 % (16-bit forward 3-14 %, fp32
//    LayerNorm backward 5-15 %).  The LayerNorm forward with fp32 weights below
//    512 lanes is the exception, and so is the 16-bit backward below 512 packs;
//  * fp32 LayerNorm forward rows of 2049..2560 packs: 512 lanes x 5 (N = 10240:
//    261 -> 222 us).
// Returns false where the general rule stands.
inline bool norm_layout(OpClass oc, int esize, int64_t packs, bool layer_norm, bool wide_weights,
                        int* G_out, int* V_out) {
  const int vp = v_pref(oc, esize);
  int G2 = pow2_ceil((packs + vp - 1) / vp);
  if (G2 < kMinG) G2 = kMinG;
  if (G2 > kMaxG) G2 = kMaxG;
  const int64_t slots = (int64_t)G2 * vp;
  if (packs > slots) return false;
  const bool fwd = oc == OC_NORM_FWD;
  const bool sparse = packs * 4 <= slots * 3;
  int G = 0, V = 0;
  if (esize == 2) {
    if (G2 == kMaxG) {
      if (sparse) {
        G = 512, V = 3;
      } else if (fwd || layer_norm) {
        G = 512, V = 4;
      }
    } else if (fwd && sparse && !(layer_norm && wide_weights && G2 < 512)) {
      // (fp32 gamma and beta beside 16-bit rows: three packs of each are 48
      // registers, and below 512 lanes the two-pack layout stays ahead)
      G = G2 / 2, V = 3;
    } else if (!fwd && sparse && G2 >= 512) {
      // the backward with three packs a lane requests its next rows ahead:
      // N = 5120: LayerNorm 95 -> 93 us, RMSNorm 92 -> 87 us; 6144: 112 -> 107 us
      // and 108 -> 102 us
      G = G2 / 2, V = 3;
    }
  } else {
    if (fwd && layer_norm && G2 == kMaxG && packs <= 2560) {
      G = 512, V = 5;
    } else if (sparse) {
      G = G2, V = 3;
    }
  }
  if (G == 0 || (int64_t)G * V < packs || !variant_built(oc, esize, G, V, true)) return false;
  *G_out = G;
  *V_out = V;
  return true;
}

// Lanes a ragged 16-bit row of `packs` packs takes in the norm forward (the rule of
// make_plan() below for such rows: two packs a lane, or three on half the lanes when
// the row fills at most three quarters of the two-pack slots), computed ahead of the
// plan because the lanes decide whether `packs` counts the row's window or the row.
inline int ragged_norm_fwd_lanes(int64_t packs, const Override& ov) {
  if (ov.G > 0) return ov.G;
  int G = pow2_ceil((packs + 1) / 2);
  if (G < kMinG) G = kMinG;
  if (G > kMaxG) G = kMaxG;
  if (ov.V == 0 && G >= 128 && packs <= (int64_t)G * 2 && packs * 4 <= (int64_t)G * 2 * 3 &&
      variant_built(OC_NORM_FWD, 2, G / 2, 3, false))
    G /= 2;
  return G;
}

// Returns 0, or -5 (ROWNORM_ERR_OVERRIDE) when a forced variant cannot hold the row.
// force_general: take the general (ragged-row) kernels even when N % E == 0.
// layer_norm: the norm op is LayerNorm (statistics of two sums, beta), not RMSNorm.
// wide_weights: fp32 gamma/beta beside 16-bit rows.
// off_line: a tensor of the call does not start on a 128-byte cache line.
// fused_add: the norm forward adds a residual row first (two rows in flight a lane);
// the norm backward adds the residual path's gradient to dX.
// masked: the softmax call reads a mask (see masked_softmax_built()).
// want_dx: the norm backward writes dX (its exact layouts exist for such calls only).
inline int make_plan(OpClass oc, int64_t M, int64_t N, int esize, int num_cus, const Override& ov,
                     bool want_cols, Plan* out, bool force_general = false,
                     bool layer_norm = false, bool wide_weights = false, bool off_line = false,
                     bool fused_add = false, bool masked = false, bool want_dx = true) {
  Plan p;
  const int E = 16 / esize;
  p.fast = (N % E) == 0 && !force_general;
  p.forced = ov.G != 0 || ov.V != 0 || ov.block != 0;
  const bool softmax = oc == OC_SOFTMAX_FWD || oc == OC_SOFTMAX_BWD;
  // the general softmax kernels address a 16-bit row through the 16-byte aligned
  // window that holds it, which starts up to E - 1 elements before the row
  int64_t packs = ((softmax && !p.fast && esize == 2 ? N + E - 1 : N) + E - 1) / E;
  // and so does the general norm forward on 256 lanes or more (norm_row_window()): the
  // lanes a row takes follow from its window's packs (halved below when three packs
  // a lane fit better, hence 512 here)
  if (oc == OC_NORM_FWD && !p.fast && esize == 2 && ov.G >= 0) {
    const int64_t wpacks = (N + E - 1 + E - 1) / E;
    if (norm_row_window(esize, ragged_norm_fwd_lanes(wpacks, ov), false)) {
      p.window = true;
      packs = wpacks;
    }
  }
  if (num_cus <= 0) num_cus = 256;
  bool stream = ov.G < 0;
  if (!stream) {
    int G, V;
    if (ov.G > 0) {
      G = ov.G;
    } else {
      G = pow2_ceil((packs + v_pref(oc, esize) - 1) / v_pref(oc, esize));
      if (G < kMinG) G = kMinG;
      if (G > kMaxG) G = kMaxG;
    }
    // GroupNorm rows of a wavefront or more (measured): about 5 packs a lane on
    // as few lanes as that allows, and exactly the packs the row has
    bool group_exact = false;
    if ((oc == OC_NORM_FWD || oc == OC_NORM_BWD) && p.fast && ov.G == 0 && ov.V == 0)
      group_exact = norm_layout(oc, esize, packs, layer_norm, wide_weights, &G, &V);
    // 16-bit forward rows of 2049..3072 packs (hidden 18432, 20480, 24576) would take
    // 1024 lanes x 3 or 4 packs, one workgroup a compute unit whose load, reduce and
    // store phases run one after the other; two 512-lane workgroups with 5 or 6 packs
    // a lane and their weights held overlap them.  Interleaved A/B at 8192 rows of
    // bf16, LayerNorm: N = 18432 121 -> 107 us (fp32 weights 122 -> 113), 20480 129 ->
    // 116 (133 -> 118), 24576 145 -> 138 (148 -> 136); 8 packs (32768) lose to 1024 x 4.
    // The RMSNorm and the fused residual add (a second row in flight) keep 1024 lanes,
    // with exactly the 3 packs such a row has (below): RMSNorm 18432 98.7 us against
    // 102.8 on 512 x 5 and 105 on 1024 x 4; add + LayerNorm 217 us against 228 on 1024 x 4.
    if (oc == OC_NORM_FWD && p.fast && esize == 2 && layer_norm && !fused_add && ov.G == 0 &&
        ov.V == 0 && packs > 2048 && packs <= 3072) {
      G = 512;
      V = packs <= 2560 ? 5 : 6;
      group_exact = true;
    }
    if (oc == OC_NORM_BWD && p.fast && ov.G == 0 && ov.V == 0 && packs > 2048 && packs <= 2560 &&
        norm_bwd_half_lanes_five(esize, wide_weights ? 4 : esize, 512, 5, !layer_norm, fused_add)) {
      G = 512;
      V = 5;
      group_exact = true;
    }
    // Norm rows of at most one wavefront of packs: with one pack a lane, a load
    // instruction of a wavefront covers one contiguous span of 64 packs (several
    // whole rows), while with V packs a lane it covers 64/G separate pieces of
    // G packs, and every piece that does not start on a cache line touches one
    // line more: 2 instead of 1 at G = 8.  Measured at 2^25 elements (fp32; rows
    // of 64 / 128 / 256 elements that start 8 bytes into a line): LayerNorm
    // forward 160 / 139 / 109 -> 105 / 104 / 105 us, backward 238 / 221 / 178 ->
    // 157 / 156 / 158 us; fp16 rows of 128 elements 78 -> 56 us and 125 -> 83 us.
    // On line-aligned rows the backward gains 4-5 % as well (its column sums take
    // a quarter of the registers), the LayerNorm forward loses 5 %: the forward
    // takes this layout for rows off the line only.
    // Softmax rows behave like the norm forward (off a line, fp32 rows of 64 / 128
    // elements: forward 130 / 138 -> 98 / 95 us, backward 172 / 198 -> 128 / 129 us;
    // on a line the forward loses 5-9 % and the backward is unchanged).
    const bool norm_or_softmax = oc == OC_NORM_FWD || oc == OC_NORM_BWD || softmax;
    if (norm_or_softmax && p.fast && ov.G == 0 && ov.V == 0 && packs <= 64 &&
        (oc == OC_NORM_BWD || off_line)) {
      G = pow2_ceil(packs);
      if (G < kMinG) G = kMinG;
      V = 1;
      group_exact = true;
    }
    // 16-bit softmax forward (its exp makes it the arithmetic-heavy one), ragged
    // 16-bit softmax rows in both directions and ragged 16-bit norm rows:
    // a row that fills at most three quarters of the two-pack slots takes three
    // packs on half the lanes (softmax N = 5120: 62 -> 56 us, 10240: 120 -> 110 us
    // at 16384 rows; at 8192 rows LayerNorm forward N = 4097: 60 -> 52 us; RMSNorm
    // backward 4097: 62 -> 55 us, 8193: 115 -> 97 us).  The ragged LayerNorm backward
    // is the exception: its three-pack kernels take 155 registers (one workgroup a
    // compute unit) where two packs on all the lanes keep two (N = 1025: 60 -> 40 us,
    // 2049: 80 -> 65 us at 16384 rows; 4097: 79 -> 66 us, 5121: 86 -> 76 us at 8192).
    const bool ragged_norm = !p.fast && (oc == OC_NORM_FWD || (oc == OC_NORM_BWD && !layer_norm));
    if (((softmax && (oc == OC_SOFTMAX_FWD || !p.fast)) || ragged_norm) &&
        esize == 2 && ov.G == 0 && ov.V == 0 &&
        G >= 128 && packs <= (int64_t)G * 2 && packs * 4 <= (int64_t)G * 2 * 3 &&
        variant_built(oc, esize, G / 2, 3, p.fast)) {
      G /= 2;
      V = 3;
      group_exact = true;
    }
    if (is_group_class(oc) && p.fast && ov.G == 0 && ov.V == 0) {
      int Gg = pow2_ceil((packs + 4) / 5);
      if (Gg > kMaxG) Gg = kMaxG;
      if (Gg >= 64) {
        int Vg = (int)((packs + Gg - 1) / Gg);
        if (Gg == kMaxG && packs <= 512 * (int64_t)group_half_lanes_max_v(oc) &&
            variant_built(oc, esize, 512, (int)((packs + 511) / 512), true)) {
          Gg = 512;
          Vg = (int)((packs + 511) / 512);
        }
        while (Vg < kMaxV && !variant_built(oc, esize, Gg, Vg, true)) ++Vg;
        if (variant_built(oc, esize, Gg, Vg, true)) {
          G = Gg;
          V = Vg;
          group_exact = true;
        }
      }
    }
    if (ov.V > 0) {
      V = ov.V;
    } else if (!group_exact) {
      V = pow2_ceil((packs + G - 1) / G);
      const int64_t v_exact = (packs + G - 1) / G;
      if (softmax && p.fast && G == kMaxG &&
          v_exact <= max_v_of(oc, esize) && variant_built(oc, esize, G, (int)v_exact, true))
        V = (int)v_exact;
      // norm backward beyond two packs a lane on 1024 lanes: norm_bwd_sums_in_lds()
      if (oc == OC_NORM_BWD && p.fast && G == kMaxG && v_exact > 2 && esize == 2)
        V = norm_bwd_lds_layout(esize, v_exact, layer_norm) ? (int)v_exact : kMaxV + 1;
      // three packs a lane at 1024 lanes, not four with a quarter of them outside the row
      if (oc == OC_NORM_FWD && p.fast && G == kMaxG && v_exact == 3 &&
          variant_built(oc, esize, G, 3, true))
        V = 3;
      // norm forward rows beyond the packs whose weights a lane holds: the next
      // pack count that is built (5, 6, 8, 10, 12, 16)
      if (oc == OC_NORM_FWD && p.fast && G == kMaxG && v_exact > kNormFwdHoldMaxV) {
        int64_t v = v_exact;
        while (v < kMaxV && !variant_built(oc, esize, G, (int)v, true)) ++v;
        V = (int)v;
        if (fused_add && V > norm_fwd_add_max_v(esize, !layer_norm)) V = kMaxV + 1;  // multi-pass
        // a handful of the longest rows: one workgroup takes 15 us for a row of 131072
        // bf16 elements, the split over workgroups 10 us for up to 64 of them (128 rows:
        // 19 us either way; rows of 65536 and fewer are faster here from 16 rows down)
        if (V >= 10 && M < num_cus / 2) V = kMaxV + 1;
      }
      if (!p.fast && V < v_pref(oc, esize)) V = v_pref(oc, esize);
    }
    // masked rows beyond 32 elements a lane at 1024 lanes: the multi-pass kernels
    if (softmax && masked && ov.V == 0 && !masked_softmax_built(esize, G, V)) V = kMaxV + 1;
    const bool holds = (int64_t)G * V >= packs;
    const int block = ov.block > 0 ? ov.block : block_threads(oc, G);
    const bool built = variant_built(oc, esize, G, V, p.fast) && block_built(oc, G, block) &&
                       !(softmax && masked && !masked_softmax_built(esize, G, V)) &&
                       !(oc == OC_NORM_BWD && p.fast &&
                         !norm_bwd_instance_ok(esize, wide_weights ? 4 : esize, G, V, !layer_norm,
                                               fused_add));
    if (ov.G > 0 || ov.V > 0 || ov.block > 0) {
      if (!holds || !built) return -5;
    }
    if (holds && built) {
      p.resident = true;
      p.G = G;
      p.V = V;
      p.block = block;
      p.rpb = p.block / G;
      // 16-bit forward rows likewise (plain calls: no residual add, no output cast)
      if (oc == OC_NORM_FWD && p.fast && !fused_add && !p.forced && ov.bpc == 0) {
        const int xi = norm_fwd_exact_index(esize, packs, M, num_cus);
        if (xi >= 0) {
          p.G = kNormFwdExact[xi].G;
          p.V = 2;
          p.block = kNormFwdExact[xi].block;
          p.rpb = p.block / p.G;
          p.exact_depth = 1;
        }
      }
      // 16-bit backward rows that fill a two-pack layout of whole wavefronts
      if (oc == OC_NORM_BWD && p.fast && want_dx && !p.forced) {
        const int xi = norm_bwd_exact_index(esize, packs, M, layer_norm, wide_weights, fused_add);
        if (xi >= 0) {
          p.G = kNormBwdExact[xi].G;
          p.V = kNormBwdExact[xi].V;
          p.block = kNormBwdExact[xi].block;
          p.rpb = p.block / p.G;
          p.exact_depth = kNormBwdExact[xi].depth;
        }
      }

    } else {
      stream = true;
    }
  }
  if (stream) {
    p.resident = false;
    p.G = kStreamBlock;
    p.V = 0;
    p.block = kStreamBlock;
    p.rpb = 1;
  }
  const int64_t nrb = (M + p.rpb - 1) / p.rpb;
  int bpc = ov.bpc > 0 ? ov.bpc : default_bpc(oc, p.block);
  // LayerNorm forward with fp32 gamma/beta beside 16-bit rows: every workgroup
  // loads twice the weight bytes, so 256-thread workgroups take half the grid
  // (16384 rows of bf16: N = 4096 53.0 -> 50.7 us, 5120 64.4 -> 62.0 us, 6144
  // 75.7 -> 73.3 us; RMSNorm and 512-thread workgroups measured no gain)
  if (ov.bpc == 0 && oc == OC_NORM_FWD && p.resident && layer_norm && wide_weights &&
      p.block == 256)
    bpc /= 2;
  // The backward that prefetches its next rows holds one workgroup a compute unit:
  // a grid of that size halves the partial rows of the dgamma/dbeta reduction
  // (bf16 [16384, 12288]: LayerNorm 222 -> 208 us, RMSNorm 210 -> 204 us)
  if (ov.bpc == 0 && oc == OC_NORM_BWD && p.resident &&
      (p.exact_depth > 0 || norm_bwd_prefetches(esize, p.G, p.V, p.fast, !layer_norm)))
    bpc = 1;
  int64_t grid = (int64_t)num_cus * bpc;
  // The norm forward beyond a few tens of thousands of rows (measured on bf16 rows
  // of 2048..8192 elements, 65536 and 262144 rows): a workgroup that walks more
  // than a handful of row blocks loses bandwidth (32 iterations: 65 % against
  // 76 %), one that walks too few reloads gamma/beta too often.  The grid grows
  // with the row count so that a workgroup makes about 2 (RMSNorm) or 4
  // (LayerNorm) iterations, twice that with fp32 weights beside 16-bit rows.
  if (oc == OC_NORM_FWD && p.resident && ov.bpc == 0) {
    const int iters = (layer_norm ? 4 : 2) * (wide_weights ? 2 : 1);
    const int64_t want = (nrb + iters - 1) / iters;
    if (grid < want) grid = want;
    // Up to a few tens of thousands of rows, fp32 weights beside 16-bit rows (and
    // LayerNorm on 512 lanes with any weights) take the other regime: three
    // 256-thread or two 512-thread workgroups a compute unit, all resident at once,
    // each walking up to 32 row blocks -- the weights are loaded once per 4..32 rows
    // and no second wave of workgroups leaves a tail.  Interleaved A/B runs, bf16
    // rows, LayerNorm with fp32 weights at 2048 / 4096 / 16384 rows: N = 4096 9.8 /
    // 17.4 / 48.9 -> 8.2 / 13.5 / 46.0 us, N = 8192 17.7 / 33.2 / 93.3 -> 14.2 / 24.3 /
    // 88.6 us; 16384 rows of 5120 / 6144: 61.2 / 72.1 -> 58.9 / 67.6 us (four
    // workgroups of 256 instead of three: 60.1 / 72.3 us).  RMSNorm with fp32 weights,
    // 16384 rows: N = 5120 56.8 -> 54.8, 7168 80.0 -> 76.0, 8192 89.3 -> 85.3, 12288
    // 135.2 -> 128.3 us.  LayerNorm with bf16 weights on 512 lanes: 7168 80.9 -> 77.4,
    // 8192 89.2 -> 86.9, 12288 136.3 -> 131.6 us (10240: 115.3 -> 117.1).  With bf16
    // weights on 256 lanes, and for RMSNorm with bf16 weights, the two regimes are
    // within 1 % at 4096-6144 and the small grid loses 3 % at 10240; the
    // residual-add forward, with twice the bytes in flight, loses 7 % on it: they
    // keep the grid above.  Rows on fewer than 256 lanes (two row slots a workgroup)
    // do not gain (N = 3072: 38.1 -> 40.0 us).  At 65536 rows and beyond (64+ row
    // blocks a workgroup) the small grid loses 3-10 %.  Grids in between (6-8
    // workgroups a compute unit, where a second wave starts) were the slowest at
    // every row count.
    if ((wide_weights || (layer_norm && p.block == 512)) && p.block <= 512 && p.rpb == 1) {
      const int64_t cap = (int64_t)num_cus * (p.block == 512 ? 2 : 3);
      if (nrb <= cap * 32) grid = cap;
    }
  }
  if (oc == OC_NORM_FWD && p.resident && p.exact_depth > 0) {
    const int xi = norm_fwd_exact_index(esize, packs, M, num_cus);
    grid = (int64_t)num_cus * kNormFwdExact[xi].bpc;
  }
  // Rows whose weights are not held gain nothing from a workgroup that walks
  // several rows: one workgroup a row (8192 rows of 40960 bf16: LayerNorm 253 ->
  // 243 us, with fp32 weights 270 -> 254 us, RMSNorm 235 -> 227 us).
  if (oc == OC_NORM_FWD && p.resident && ov.bpc == 0 &&
      !norm_fwd_holds_weights(esize, wide_weights ? 4 : esize, p.G, p.V, p.fast, !layer_norm,
                              fused_add))
    grid = nrb;
  if (!p.resident) p.window = false;
  // windowed rows: 1024 threads a compute unit, all resident at once, so that a
  // workgroup loads its shifted weights once for all its rows (fp16 [8192, 4097]
  // LayerNorm: 4 workgroups of 256 a compute unit 34.6 us, 2: 45.9, 8: 40.0, one row a
  // workgroup 52.3; [8192, 8193] on 512 threads: 2 a compute unit 61.0 us, 1: 83.9, 4: 69.5)
  if (p.window && ov.bpc == 0) grid = (int64_t)num_cus * (1024 / p.block);
  if (grid > nrb) grid = nrb;
  if (grid > 0x7fffffff) grid = 0x7fffffff;
  if (grid < 1) grid = 1;
  // (the kernel takes the window from its lanes: the two must agree)
  if (p.resident && oc == OC_NORM_FWD && p.window != norm_row_window(esize, p.G, p.fast)) return -5;
  // windowed rows: a workgroup that walks several row blocks strides by a multiple of
  // 8 rows, so that every row of a lane group has the same window head
  if (p.window && grid < nrb && grid % 8 != 0) grid = grid > 8 ? grid - grid % 8 : (nrb < 8 ? nrb : 8);
  p.grid = grid;
  p.partial_rows = 0;
  if (oc == OC_NORM_BWD && want_cols) {
    // resident: one partial row per workgroup; streaming: a separate column-sum
    // kernel whose grid.y is the partial-row count.
    if (p.resident) {
      p.partial_rows = grid;
    } else {
      // enough partial rows that the column-sum grid (256 lanes, one pack each,
      // across; partial rows down) gives a compute unit about four workgroups
      const int64_t across = (packs + 255) / 256;
      int64_t pr = (4 * (int64_t)num_cus + across - 1) / across;
      if (pr > 64) pr = 64;
      // rows so long that the columns alone give every compute unit two workgroups: one
      // partial row, which the column-sum kernels then write as dgamma / dbeta themselves
      // (no second stage; bf16 LayerNorm backward [2, 1310720] 25.8 -> 13.9 us, [16, 1048576] 40.7 ->
      // 34.1 us)
      if (across >= 2 * (int64_t)num_cus) pr = 1;
      if (pr > M) pr = M;
      p.partial_rows = pr < 1 ? 1 : pr;
    }
  }
  // Rows beyond the registers, and too few of them to give every compute unit a
  // workgroup (the regime of the reference's split-row kernels, Norm.h:632-812):
  // cut each row into chunks so that about four workgroups per compute unit
  // exist.  The partial sums of a row cross workgroups through memory, in a fixed
  // order, between two launches.
  if ((oc == OC_NORM_FWD || oc == OC_NORM_BWD) && !p.resident) {
    const int64_t min_chunk = (int64_t)kSplitMinStrides * kStreamBlock;
    int64_t want = 1;
    if (ov.G < 0 && ov.V > 0)
      want = ov.V;
    else if (M > 0 && M < 2 * (int64_t)num_cus)
      want = (4 * (int64_t)num_cus + M - 1) / M;
    if (want > kSplitMaxChunks) want = kSplitMaxChunks;
    if (want > 1) {
      int64_t cp = (packs + want - 1) / want;
      cp = (cp + kStreamBlock - 1) / kStreamBlock * kStreamBlock;
      if (cp < min_chunk && !(ov.G < 0 && ov.V > 0)) cp = min_chunk;
      int64_t chunks = (packs + cp - 1) / cp;
      // a remainder of less than one workgroup stride joins the chunk before it, so
      // every chunk holds at least kStreamBlock packs (the forward keeps a chunk's
      // partial sums in the first bytes of the chunk's own output)
      if (chunks > 1 && packs - (chunks - 1) * cp < kStreamBlock) --chunks;
      if (chunks > 1) {
        p.split = (int)chunks;
        p.chunk_packs = cp;
      }
    }
  }
  // Forward rows beyond one workgroup's registers: a team of workgroups holds the
  // row (one pass over X).  As few workgroups a row as hold it with 16 packs a lane,
  // then as many teams as there are rows and compute units, and a row spread over
  // all the workgroups its team can have (down to one stride of 1024 packs each).
  // (GroupNorm forward slabs likewise; the caller takes the team only where the channels
  // are whole packs)
  // (also rows that one workgroup still holds, 16 packs a lane on 1024 lanes, when there are
  // too few of them for the compute units: bf16 [128, 131072] LayerNorm 17.4 -> 13.8 us, fp32
  // [128, 65536] 19.2 -> 13.3 us; from 8192 packs down the resident kernel is as fast or faster,
  // its 4-6 us against the team's 6-8)
  const bool few_rows = oc == OC_NORM_FWD && p.resident && 2 * M <= num_cus &&
                        packs >= (int64_t)kMaxG * kMaxV;
  if ((oc == OC_NORM_FWD || oc == OC_GROUP_FWD) && (!p.resident || few_rows) && p.fast && !fused_add &&
      ov.G == 0 && ov.V == 0 && ov.bpc == 0 && ov.block == 0) {
    const int64_t cus = num_cus * kTeamPerCu < kTeamMaxWorkgroups ? num_cus * kTeamPerCu : kTeamMaxWorkgroups;
    const int64_t per_wg = (int64_t)kTeamBlock * kTeamMaxV;
    const int64_t team_min = (packs + per_wg - 1) / per_wg;
    int64_t teams = team_min <= cus ? cus / team_min : 0;
    if (teams > M) teams = M;
    // Fewer than 8 teams run their load, wait and store phases nearly in step, and
    // the wait (about 8 us a round) is not hidden by other teams: bf16 [128, 9834496]
    // (3 teams of 85, 43 rounds) took 1740 us against 1500 us for the two-pass kernel
    // whose second pass comes out of the memory-side cache, [2, 1310720] 13.2 against
    // 11.6 us; 8 teams ([8, 4194304], one round) 35.1 against 40.5 us, 64 teams
    // ([512, 401408], 8 rounds) 177 against 196 us.
    // (GroupNorm slabs have no split-row kernels to fall back on: with fewer slabs than 8
    // teams, all at once, the alternative is one workgroup a slab)
    if (teams >= kTeamMinTeams || ((oc == OC_GROUP_FWD || few_rows) && teams >= 1 && teams == M)) {
      // a chunk is a whole number of workgroup strides, exactly the packs a lane the
      // kernel is compiled for: every workgroup but a row's last runs straight-line code
      int64_t team_max = cus / teams;
      const int64_t strides = (packs + kTeamBlock - 1) / kTeamBlock;
      if (team_max > strides) team_max = strides;
      const int64_t v = (strides + team_max - 1) / team_max;
      const int64_t team = (strides + v - 1) / v;
      p.team = (int)team;
      p.team_v = (int)v;
      p.team_chunk_packs = v * kTeamBlock;
      p.team_grid = teams * team;
    }
  }
  // Forward rows too long for at least eight such teams (beyond 256 / 8 * 16 * 512 packs),
  // many of them, weights no wider than the rows: one team over the machine, one workgroup a
  // compute unit, kTeamFwdLongPacks packs a lane, three rows in flight a workgroup and gamma /
  // beta held for the whole call (norm_fwd_rows_team_kernel).
  // (override G = -1 with block = 1: whatever the rounds and the other teams, for tests)
  const bool team_rows_forced = ov.G == -1 && ov.V == 0 && ov.block == 1 && ov.bpc == 0;
  if (oc == OC_NORM_FWD && !p.resident && p.fast && !fused_add && !wide_weights &&
      ((ov.G == 0 && ov.V == 0 && ov.bpc == 0 && ov.block == 0 && p.team == 0) || team_rows_forced)) {
    const int64_t cus = num_cus < kTeamMaxWorkgroups ? num_cus : kTeamMaxWorkgroups;
    const int64_t chunk = (int64_t)kTeamFwdLongPacks * kTeamBlock;
    const int64_t team = (packs + chunk - 1) / chunk;
    if (team >= 2 && team <= cus) {
      int64_t teams = cus / team;
      if (teams > M) teams = M;
      const bool rounds_ok = M >= kTeamFwdMinRounds * teams;
      const bool full_ok = 5 * packs >= 4 * team * chunk;
      if (teams >= 1 && ((rounds_ok && full_ok) || team_rows_forced)) {
        p.team = (int)team;
        p.team_v = kTeamFwdLongPacks;
        p.team_r = 1;
        p.team_chunk_packs = chunk;
        p.team_grid = teams * team;
      }
    }
  }
  // Backward rows beyond one workgroup's registers (whole packs, dX wanted, no residual
  // gradient): teams of workgroups hold kTeamBwdRows rows at a time, kTeamBwdPacks strides of
  // packs a workgroup, dY and X read once (norm_bwd_team_kernel).
  // (override G = -1 with block = 1: the team launch whatever the rounds, for tests)
  const bool team_bwd_forced = ov.G == -1 && ov.V == 0 && ov.block == 1 && ov.bpc == 0;
  if (oc == OC_NORM_BWD && !p.resident && p.fast && !fused_add && want_dx &&
      ((ov.G == 0 && ov.V == 0 && ov.bpc == 0 && ov.block == 0) || team_bwd_forced)) {
    const int64_t cus = num_cus * kTeamBwdPerCu < kTeamMaxWorkgroups ? num_cus * kTeamBwdPerCu : kTeamMaxWorkgroups;
    const int64_t chunk = (int64_t)kTeamBwdPacks * kTeamBlock;
    const int64_t team = (packs + chunk - 1) / chunk;
    const int64_t ngroups = (M + kTeamBwdRows - 1) / kTeamBwdRows;
    if (team >= 2 && team <= cus) {
      int64_t teams = cus / team;
      if (teams > ngroups) teams = ngroups;
      // Worth it from the second round on (a call costs about 25 us beside 9.5-10 us a round,
      // where the two passes of the other kernels cost about 14.6 us for a round's rows); a
      // LayerNorm on large teams (more than 64 workgroups a row) from the fourth.  Measured,
      // bf16, LayerNorm / RMSNorm, team against two passes in us: [512, 401408] (26 rounds)
      // 258 / 243 against 359 / 350; [4096, 65536] (64) 330 / 308 against 478 / 468; [100,
      // 401408] (5) 66 / 59 against 80 / 75; [1024, 40960] (5) 82 / 72 against 81 / 75; [512,
      // 65536] (4) 62 / 52 against 68 / 63; [32, 401408] (2) 34 / 29 against 41 / 37; [64,
      // 262144] (2) 41 / 32 against 41 / 38; [16, 1048576] (2, 128 workgroups a row) 41 / 31
      // against 35 / 34; [8192, 24584] (a row's last workgroup holds a single pack) 327
      // against 380.
      const bool rounds_ok = layer_norm && team > 64 ? ngroups >= 4 * teams : ngroups > teams;
      if (teams >= 1 && (rounds_ok || team_bwd_forced)) {
        p.team = (int)team;
        p.team_v = kTeamBwdPacks;
        p.team_chunk_packs = chunk;
        p.team_grid = teams * team;
        p.team_partial_rows = want_cols ? teams : 0;
      }
    }
  }
  // Softmax forward / backward of few, very long rows of whole packs: one workgroup a row
  // would leave most compute units idle, so each row is held by a team of workgroups
  // (softmax_fwd_team_kernel / softmax_bwd_team_kernel): as few workgroups a row as hold it
  // with 16 (backward: 8 of each tensor) packs a lane, then as many teams as there are rows
  // and room, and a row spread over all the workgroups its team can have.  More rows than
  // teams run in rounds; even then, and with few teams whose waits nothing hides, one
  // workgroup a row is several times slower (fp32 [2, 16777216]: 4800 us).
  if (softmax && p.fast && !masked && ov.G == 0 && ov.V == 0 && ov.bpc == 0 && ov.block == 0 &&
      2 * M <= num_cus && packs >= kSoftmaxTeamMinPacks) {
    const int64_t cus = num_cus * kTeamPerCu < kTeamMaxWorkgroups ? num_cus * kTeamPerCu : kTeamMaxWorkgroups;
    const int max_v = oc == OC_SOFTMAX_FWD ? kTeamMaxV : kSoftmaxBwdTeamMaxV;
    const int64_t per_wg = (int64_t)kTeamBlock * max_v;
    const int64_t team_min = (packs + per_wg - 1) / per_wg;
    int64_t teams = team_min <= cus ? cus / team_min : 0;
    if (teams > M) teams = M;
    if (teams >= 1) {
      int64_t team_max = cus / teams;
      const int64_t strides = (packs + kTeamBlock - 1) / kTeamBlock;
      if (team_max > strides) team_max = strides;
      const int64_t v = (strides + team_max - 1) / team_max;
      const int64_t team = (strides + v - 1) / v;
      if (team >= 2) {
        p.team = (int)team;
        p.team_v = (int)v;
        p.team_chunk_packs = v * kTeamBlock;
        p.team_grid = teams * team;
      }
    }
  }
  if (oc == OC_SOFTMAX_BWD && !p.resident && p.fast && ov.G == 0 &&
      packs <= (int64_t)kMaxG * kGradResidentMaxV)
    p.grad_resident = true;
  *out = p;
  return 0;
}

// ---- softmax over a non-innermost dimension: [outer, D, inner] ----------------
//
// A group of TX * TY threads owns one tile: TX lanes along `inner` (one 16-byte
// pack each) by TY threads along D, each holding V packs, so the registers
// cover D <= TY * V rows.  The rule: at most 8 packs a lane (4 for the 16-bit
// backward of D <= 32), TY = the power of two that then covers D, V = ceil(D / TY), and TX = as many lanes
// as a row of `inner` has packs, capped so that a group is one wavefront where
// that leaves at least 8 lanes (128-byte segments) per row, and 256 threads
// otherwise.  A group of one wavefront reduces with shuffles alone.  D beyond
// 64 rows x 8 packs x 4 lanes takes the multi-pass kernel.
struct StridedPlan {
  bool resident = true;
  bool fast = true;  // inner % E == 0
  int tx_log2 = 0, ty_log2 = 0, V = 0, block = 0;
  int64_t grid = 0;
  // multi-pass kernels with too few tiles for the machine: the D rows are cut into
  // `chunks` chunks of `chunk_rows` rows, one workgroup each (0 or 1: not split)
  int chunks = 0, chunk_rows = 0;
};

constexpr int kStridedSplitUnroll = 4;  // rows a lane of the split kernels requests at a time

constexpr int kStridedBlock = 256;
constexpr int kStridedMaxV = 8;

inline int log2_of_pow2(int v) {
  int l = 0;
  while ((1 << l) < v) ++l;
  return l;
}

// Override: G = lanes along inner (power of two 1..64; -1 forces the multi-pass
// kernel, and then V = 1 keeps all D rows of a tile on one workgroup, V > 1 cuts
// them into that many chunks), V = packs per lane.  Returns 0 or -5.
inline int make_strided_plan(bool backward, int64_t outer, int64_t D, int64_t inner, int esize,
                             int num_cus, const Override& ov, StridedPlan* out) {
  StridedPlan p;
  const int E = 16 / esize;
  const int64_t packs = (inner + E - 1) / E;
  p.fast = (inner % E) == 0;
  p.block = kStridedBlock;
  // an empty tensor launches nothing (the entry points return before they plan; the
  // plan query gets a plan with no workgroups)
  if (outer < 1 || D < 1 || inner < 1) {
    *out = p;
    return 0;
  }
  if (num_cus <= 0) num_cus = 256;
  const int px = packs >= 64 ? 64 : pow2_ceil(packs);  // lanes a row of `inner` can use
  // packs a lane may hold: 8, or 4 for the 16-bit backward (two packed rows per
  // lane) while a wavefront still covers D -- measured faster
  int vcap = kStridedMaxV;
  if (backward && esize == 2 && D > 4 && D <= 32) vcap = 4;
  if (ov.V > 0 && ov.G >= 0) vcap = ov.V;
  if (vcap < 1 || vcap > kStridedMaxV) return -5;
  // TY = the power of two that covers D with at most vcap rows a thread; V = the
  // rows a thread then really has (not rounded up: D = 21 is 4 x 6, not 4 x 8)
  const int64_t ty_need = pow2_ceil((D + vcap - 1) / vcap);
  int V = (ov.V > 0 && ov.G >= 0) ? ov.V : (int)((D + ty_need - 1) / ty_need);
  int TX = 0, TY = 0;
  // rows are never cut below 4 lanes (64 bytes) to make room for a larger D
  const int ty_max = kStridedBlock / (px < 4 ? px : 4);
  bool stream = ov.G < 0 || (ov.G == 0 && ty_need > ty_max) || ty_need > kStridedBlock;
  if (!stream) {
    TY = (int)ty_need;
    if (ov.G > 0) {
      if (ov.G > 64 || (ov.G & (ov.G - 1))) return -5;
      TX = ov.G;
    } else {
      int cap = 64 / TY;                 // one wavefront per group ...
      if (cap < 8) cap = 8;              // ... unless rows would shrink below 128 bytes
      if (cap * TY > kStridedBlock) cap = kStridedBlock / TY;
      TX = px < cap ? px : cap;
    }
    if ((int64_t)TX * TY > kStridedBlock || TX < 1) {
      if (ov.G > 0 || ov.V > 0) return -5;
      stream = true;
    }
  } else if (ov.G > 0 || (ov.V > 0 && ov.G >= 0)) {
    return -5;
  }
  if (stream) {
    // one group per workgroup, rows of up to 16 lanes (256 bytes; [8192, 8192] over dim 0,
    // forward / backward: 8 lanes 81.6 / 120.9 us, 16 lanes 80.1 / 113.9, 32 lanes 84.2 / 115.2)
    TX = px < 16 ? px : 16;
    TY = kStridedBlock / TX;
    V = 0;
    // Too few tiles to fill the machine (softmax over dim 0 of [8192, 8192] is 128
    // tiles): cut the D rows into chunks of whole TY * unroll strides so that
    // about four workgroups per compute unit exist; a short remainder joins the
    // chunk before it.
    const int64_t tiles = outer * ((packs + TX - 1) / TX);
    const int64_t min_rows = (int64_t)TY * kStridedSplitUnroll;
    int64_t want = 1;
    if (ov.G < 0 && ov.V > 0)
      want = ov.V;
    else if (tiles < 2 * (int64_t)num_cus)
      want = (4 * (int64_t)num_cus + tiles - 1) / tiles;
    if (want > 1) {
      int64_t rows = (D + want - 1) / want;
      rows = (rows + TY - 1) / TY * TY;
      if (rows < min_rows && !(ov.G < 0 && ov.V > 0)) rows = min_rows;
      int64_t chunks = (D + rows - 1) / rows;
      if (chunks > 1 && D - (chunks - 1) * rows < TY) --chunks;
      if (chunks > 65535) chunks = 1;
      if (chunks > 1) {
        p.chunks = (int)chunks;
        p.chunk_rows = (int)rows;
      }
    }
    if (p.chunks <= 1 && !(ov.G < 0 && ov.V > 0)) {
      // not split: fewer lanes along inner while the problem has less than two
      // workgroups per compute unit
      while (TX > 4 && outer * ((packs + TX - 1) / TX) < 2 * (int64_t)num_cus) TX >>= 1;
      TY = kStridedBlock / TX;
    }
  }
  p.resident = !stream;
  p.tx_log2 = log2_of_pow2(TX);
  p.ty_log2 = log2_of_pow2(TY);
  p.V = V;
  const int64_t xtiles = (packs + TX - 1) / TX;
  const int64_t ntiles = outer * xtiles;
  const int groups = kStridedBlock / (TX * TY);
  const int64_t nblocks = (ntiles + groups - 1) / groups;
  const int bpc = ov.bpc > 0 ? ov.bpc : (1 << 20);
  int64_t grid = (int64_t)num_cus * bpc;
  if (grid > nblocks) grid = nblocks;
  if (grid > 0x7fffffff) grid = 0x7fffffff;
  if (grid < 1) grid = 1;
  p.grid = grid;
  *out = p;
  return 0;
}

}  // namespace rownorm
