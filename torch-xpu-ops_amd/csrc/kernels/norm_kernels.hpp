// LayerNorm / RMSNorm forward and backward kernels for gfx950 (wave64).
//
// Layout of one call: the input is a dense [M, N] matrix.  G lanes share one
// row; lane l of the group owns the 16-byte packs number l, l+G, l+2G, ...
// (V of them), so each wave-wide access covers one contiguous kilobyte.  A
// workgroup of BLOCK threads handles BLOCK/G rows per iteration and strides
// over the rows persistently, which lets the per-column quantities (gamma,
// beta, and in the backward pass the dgamma/dbeta partial sums) stay in
// registers from the first row to the last.  Forward rows of more packs a lane
// than the registers hold beside their weights (norm_fwd_holds_weights() in
// plan.hpp: 16-bit rows beyond 32768 elements, up to 131072) keep only the row and
// read gamma / beta, which stay in L2, where the output needs them; backward rows
// of three or four 16-bit packs a lane on 1024 lanes (norm_bwd_sums_in_lds():
// 16392..32768 elements) keep their dgamma sums in LDS and gamma in L2.
//
// What these kernels stand in for in the reference (the arithmetic, not the
// code shape):
//   forward   VectorizedLayerNormKernelFunctor + compute_stats,
//             src/ATen/native/xpu/sycl/LayerNormKernels.cpp:394-586, and the
//             scalar pair RowwiseMomentsFunctor / LayerNormForwardKernelFunctor
//             (:203-320) used for unaligned pointers or N % 4 != 0;
//   backward  FusedNormKernelFunctor (src/ATen/native/xpu/sycl/Norm.h:485-526)
//             with LayerNormBackward::reduce_combine/update
//             (LayerNormKernels.cpp:86-186) for dX, and
//             GammaBetaBackwardSimpleKernelFunctor (:885-1024) /
//             GammaBetaReduceFunctor (:709-874) + at::sum (:1312-1314) for
//             dgamma/dbeta.
// Differences by design: X and dY are read once (the reference reads them
// twice for dX and a third time for dgamma/dbeta); the column partial sums
// are fp32 whatever the weight dtype; every access is 128 bits wide for any
// pointer alignment; the weight dtype is independent of the row dtype.
#pragma once
#include <type_traits>

#include "device/flat_rows.hpp"
#include "device/pack.hpp"
#include "plan.hpp"
#include "device/reduce.hpp"
#include "device/team.hpp"

namespace rownorm {

// ---------------------------------------------------------------------------
// Forward, row resident in registers: one read of X, one write of Y.
//
// LayerNorm statistics: mean0 = sum(x)/N, then the centred sums
// s1 = sum(x - mean0), s2 = sum((x - mean0)^2) over the registers give
// mean = mean0 + s1/N and var = (s2 - s1*s1/N)/N.  On a constant row the
// correction cancels the rounding of mean0 exactly, so mean is the constant
// and y is beta bit for bit, which is what the CPU kernel's Welford pass gives
// (Welford recurrence being followed: src/ATen/native/xpu/sycl/
// SharedReduceOps.h:56-88).
//
// FAST: N is a whole number of packs (see row_load in device/pack.hpp).
// R: rows each lane group works on per iteration; their loads are issued
// together and their sums share one reduction (one barrier for R rows).  The
// library is built with R = 1: on MI355X R = 2 measured only 1-3% faster at
// G >= 256 (and slower in the backward, whose two-row body needs over 150
// VGPRs), not worth twice the kernels.
//
// ADD: the row that is normalized is h = x + res (the residual stream of a
// transformer block), formed in float32 and rounded once to T, exactly what an
// elementwise add of the two tensors gives; h is written out (one read of x,
// one of res, one write of h and one of y instead of the three reads and two
// writes of an add followed by a norm).  h may be the memory of x or of res: a
// lane stores its h packs after the statistics, when every lane of the row has
// read what it needs.  TY: the element type of y (the output cast fused into the
// store; T unless a float32 row is written out in 16 bits).
template <class T, class WT, int G, int V, int BLOCK, int R, bool RMS, bool FAST, class TY = T,
          bool ADD = false>
__global__ void __launch_bounds__(BLOCK)
norm_fwd_resident_kernel(const T* __restrict__ x, const T* res, const WT* __restrict__ gamma,
                         const WT* __restrict__ beta, T* h, TY* __restrict__ y,
                         float* __restrict__ mean, float* __restrict__ rstd, int64_t M, int N,
                         float eps) {
  constexpr int E = elems_per_pack<T>::value;
  constexpr int RPB = BLOCK / G;  // row slots of the workgroup
  constexpr int RPI = RPB * R;    // rows per workgroup iteration
  __shared__ float red[reduce_lds_floats<G, BLOCK, 2 * R>::value];
  int phase = 0;
  const int slot = threadIdx.x / G;
  const int lane0 = threadIdx.x % G;
  const float fN = (float)N;
  const float inv_n = 1.0f / fN;

  // gamma/beta of this lane's columns stay in registers for all rows: widened to
  // fp32 once when they are few, otherwise in storage format and widened per row.
  // Rows of more packs a lane than norm_fwd_holds_weights() allows leave them in
  // memory and load each pack of them (from L2) where the output needs it.
  constexpr bool kWideWeights = V * E <= 16;
  constexpr bool kHold =
      norm_fwd_holds_weights((int)sizeof(T), (int)sizeof(WT), G, V, FAST, RMS, ADD);
  const bool exact = N == G * V * E;  // every pack of every lane lies inside the row
  // WINDOW (norm_row_window()): ragged 16-bit rows are addressed through the 16-byte
  // aligned window that holds the row, `hd` elements ahead of it; the held weights
  // are those of the window's columns and are loaded again should a row of this lane
  // group sit at another head (the planner's grids keep it constant).
  constexpr bool WINDOW = norm_row_window((int)sizeof(T), G, FAST);
  static_assert(!WINDOW || (R == 1 && kHold), "windowed rows: one row a lane group, weights held");
  Pack<WT, E> gp[kHold ? V : 1];
  Pack<WT, E> bp[RMS || !kHold ? 1 : V];
  auto load_weights = [&](int head) {
#pragma unroll
    for (int c = 0; c < V; ++c) {
      const int e0 = (c * G + lane0) * E - head;
      gp[kHold ? c : 0] = gamma ? load_row_pack<WT, E, false>(gamma, e0, N, true, 1.0f)
                                : Pack<WT, E>::splat(1.0f);
      if constexpr (!RMS)
        bp[kHold ? c : 0] =
            beta ? load_row_pack<WT, E, false>(beta, e0, N, true, 0.0f) : Pack<WT, E>::zero();
    }
  };
  int held_head = -1;
  if constexpr (kHold && !WINDOW) load_weights(0);

  const int64_t nrb = (M + RPI - 1) / RPI;
  for (int64_t rb = blockIdx.x; rb < nrb; rb += gridDim.x) {
    const int64_t row0 = (rb * RPB + slot) * R;
    // (many packs a lane: their offsets are formed where they are used, not held)
    const int lane = lane_again<!kHold>(lane0);
    bool ok[R];
    Pack<T, E> xp[R][V];
    int hd = 0;  // the window's head; N + hd: the row's end in window elements
    if constexpr (WINDOW) {
      hd = window_head<T, E>(x + ((RPI == 1 || row0 < M) ? row0 : 0) * (int64_t)N);
      if (hd != held_head) {
        load_weights(hd);
        held_head = hd;
      }
    }
    const int nw = N + hd;
#pragma unroll
    for (int r = 0; r < R; ++r) {
      ok[r] = (RPI == 1) ? true : row0 + r < M;
      const T* xr = x + (ok[r] ? row0 + r : 0) * (int64_t)N - hd;
#pragma unroll
      for (int c = 0; c < V; ++c)
        xp[r][c] = row_load<T, E, true, FAST>(xr, (c * G + lane) * E, nw, ok[r], 0.0f, hd, WINDOW);
      if constexpr (ADD) {
        const T* rr = res + (ok[r] ? row0 + r : 0) * (int64_t)N - hd;
        Pack<T, E> rp[V];
#pragma unroll
        for (int c = 0; c < V; ++c)
          rp[c] = row_load<T, E, true, FAST>(rr, (c * G + lane) * E, nw, ok[r], 0.0f, hd, WINDOW);
#pragma unroll
        for (int c = 0; c < V; ++c)
#pragma unroll
          for (int i = 0; i < E; ++i) xp[r][c].set(i, xp[r][c].get(i) + rp[c].get(i));
      }
      // (the RMSNorm sums squares: the window's elements outside the row become zero;
      // the LayerNorm replaces them by its centre below)
      if constexpr (WINDOW && RMS) {
#pragma unroll
        for (int c = 0; c < V; ++c)
          row_trim<T, E, FAST>(xp[r][c], (c * G + lane) * E, nw, 0.0f, hd, WINDOW);
      }
    }

    float mean0[R], m1[R], rs[R];
    if constexpr (RMS) {
      float acc[R];
#pragma unroll
      for (int r = 0; r < R; ++r) {
        acc[r] = 0.0f;
#pragma unroll
        for (int c = 0; c < V; ++c)
#pragma unroll
          for (int i = 0; i < E; ++i) {
            const float v = xp[r][c].get(i);
            acc[r] = fmaf(v, v, acc[r]);
          }
      }
      group_allreduce<G, BLOCK, R, SumOp>(acc, red, phase);
#pragma unroll
      for (int r = 0; r < R; ++r) {
        rs[r] = row_rstd_of<T>(row_mean_of<T>(acc[r], fN, inv_n) + eps);
        mean0[r] = m1[r] = 0.0f;
      }
    } else if constexpr (sizeof(T) == 2) {
      // 16-bit rows: one reduction round.  Every lane of the row centres on the
      // same value k, the median of the row's first three elements (one 16-byte
      // load of the same address for all lanes), and sums (x - k), (x - k)^2:
      // mean = k + s1/N, var = (s2 - s1*s1/N)/N.  The subtraction only cancels
      // when k is far from the row against its spread, i.e. two of the first
      // three elements are outliers, and even then the error stays inside the
      // 16-bit tolerance; fp32 rows keep the two-round form below, which is
      // exact for any data.  On a constant row x - k is exactly zero, so y is
      // beta bit for bit here too.
      float acc[2 * R];
#pragma unroll
      for (int r = 0; r < R; ++r) {
        const T* xr = x + (ok[r] ? row0 + r : 0) * (int64_t)N;
        Pack<T, E> head = load_row_pack<T, E, false>(xr, 0, N, true, 0.0f);
        if constexpr (ADD) {
          // the head of h, formed as the lane that owns it forms it
          const Pack<T, E> rh = load_row_pack<T, E, false>(
              res + (ok[r] ? row0 + r : 0) * (int64_t)N, 0, N, true, 0.0f);
#pragma unroll
          for (int i = 0; i < 3; ++i) head.set(i, head.get(i) + rh.get(i));
        }
        const float a = head.get(0), b = head.get(1), c3 = head.get(2);
        const float k = fmaxf(fminf(a, b), fminf(fmaxf(a, b), c3));
        mean0[r] = k;
        acc[2 * r] = acc[2 * r + 1] = 0.0f;
        if constexpr (FAST) {
          // a pack lies wholly inside or wholly outside the row: the ones outside
          // become k (a value of the row, so exact in T) and add nothing
          if (!exact) {
            const Pack<T, E> kp = Pack<T, E>::splat(k);
#pragma unroll
            for (int c = 0; c < V; ++c)
              if ((c * G + lane) * E >= N) xp[r][c] = kp;
          }
        }
        if constexpr (!FAST) {
          // ragged rows: the elements past the row end (the tail of its last pack, the
          // packs beyond it, a row slot past the last row) become k likewise, under a
          // branch that only their lanes take, instead of a select per element (fp16
          // rows of 2047: 41 -> 38.5 us at 16384 rows, of 257: 35 -> 32.4 us at 65536)
#pragma unroll
          for (int c = 0; c < V; ++c) {
            const int nvalid = ok[r] ? nw - (c * G + lane) * E : 0;
            const int nahead = WINDOW ? hd - (c * G + lane) * E : 0;  // (the window's first pack)
            if (nvalid < E || nahead > 0) {
#pragma unroll
              for (int i = 0; i < E; ++i)
                if (i >= nvalid || i < nahead) xp[r][c].set(i, k);
            }
          }
        }
#pragma unroll
        for (int c = 0; c < V; ++c) {
#pragma unroll
          for (int i = 0; i < E; ++i) {
            const float d = xp[r][c].get(i) - k;
            acc[2 * r] += d;
            acc[2 * r + 1] = fmaf(d, d, acc[2 * r + 1]);
          }
        }
      }
      group_allreduce<G, BLOCK, 2 * R, SumOp>(acc, red, phase);
#pragma unroll
      for (int r = 0; r < R; ++r) {
        m1[r] = row_mean_of<T>(acc[2 * r], fN, inv_n);
        float var = row_mean_of<T>(acc[2 * r + 1] - acc[2 * r] * m1[r], fN, inv_n);
        var = var < 0.0f ? 0.0f : var;  // a select, not v_max_f32: a NaN row keeps NaN statistics
        rs[r] = row_rstd_of<T>(var + eps);
      }
    } else {
      float acc0[R];
#pragma unroll
      for (int r = 0; r < R; ++r) {
        acc0[r] = 0.0f;
#pragma unroll
        for (int c = 0; c < V; ++c)
#pragma unroll
          for (int i = 0; i < E; ++i) acc0[r] += xp[r][c].get(i);
      }
      group_allreduce<G, BLOCK, R, SumOp>(acc0, red, phase);
      float acc[2 * R];
      // MASKED: some packs reach past the row end; their elements must not count.
#pragma unroll
      for (int r = 0; r < R; ++r) mean0[r] = acc0[r] / fN;
      auto centred_sums = [&](auto masked) {
        constexpr bool MASKED = decltype(masked)::value;
#pragma unroll
        for (int r = 0; r < R; ++r) {
          acc[2 * r] = acc[2 * r + 1] = 0.0f;
#pragma unroll
          for (int c = 0; c < V; ++c) {
            keep_packed(xp[r][c]);
            const int nvalid = ok[r] ? N - (c * G + lane) * E : 0;  // elements inside the row
#pragma unroll
            for (int i = 0; i < E; ++i) {
              float d = xp[r][c].get(i) - mean0[r];
              if constexpr (MASKED) d = (i < nvalid) ? d : 0.0f;
              acc[2 * r] += d;
              acc[2 * r + 1] = fmaf(d, d, acc[2 * r + 1]);
            }
          }
        }
      };
      if (exact) {
        centred_sums(std::false_type{});
      } else if constexpr (FAST && sizeof(T) == 4) {
        // a pack lies wholly inside or wholly outside the row: the ones outside
        // become mean0 and add nothing
#pragma unroll
        for (int r = 0; r < R; ++r)
#pragma unroll
          for (int c = 0; c < V; ++c)
            if ((c * G + lane) * E >= N) xp[r][c] = Pack<T, E>::splat(mean0[r]);
        centred_sums(std::false_type{});
      } else {
        centred_sums(std::true_type{});
      }
      group_allreduce<G, BLOCK, 2 * R, SumOp>(acc, red, phase);
#pragma unroll
      for (int r = 0; r < R; ++r) {
        m1[r] = row_mean_of<T>(acc[2 * r], fN, inv_n);
        float var = row_mean_of<T>(acc[2 * r + 1] - acc[2 * r] * m1[r], fN, inv_n);
        var = var < 0.0f ? 0.0f : var;  // a select, not v_max_f32: a NaN row keeps NaN statistics
        rs[r] = row_rstd_of<T>(var + eps);
      }
    }

    // y = gamma * (rstd * (x - mean)) + beta with x - mean taken as (x - mean0) - m1:
    // both differences are exact where it matters (constant rows give beta bit for
    // bit) and the rounding of mean0 + m1 to one float never enters y.  (Keeping
    // x - mean0 in fp32 registers from the previous pass would save two VALU ops an
    // element; it measured slower: fewer wavefronts stay resident.)
    float nm1rs[R];
#pragma unroll
    for (int r = 0; r < R; ++r) nm1rs[r] = -m1[r] * rs[r];
    const int ls = lane_after<!kHold>(lane0, nm1rs[0]);
#pragma unroll
    for (int r = 0; r < R; ++r) {
      TY* yr = y + (row0 + r) * (int64_t)N - hd;
      // Weights that are not held (rows of whole packs only) are looked up with plain
      // loads, pack c + 1 before pack c is stored.  A test of the pointer would be a
      // branch around the load, whose join waits for every request outstanding, and
      // requests complete in order: a lookup issued behind a store waits for that store.
      // An absent weight is read from the head of X (such a row is long enough) and
      // replaced.
      auto lookup = [&](const WT* w, int c, float dflt) {
        const bool have = w != nullptr;
        Pack<WT, E> p = row_load<WT, E, false, true>(
            have ? w : reinterpret_cast<const WT*>(x), have ? (c * G + ls) * E : 0, N, true, dflt);
        if (!have) p = Pack<WT, E>::splat(dflt);
        return p;
      };
      Pack<WT, E> gahead, bahead;
      if constexpr (!kHold) {
        gahead = lookup(gamma, 0, 1.0f);
        if constexpr (!RMS) bahead = lookup(beta, 0, 0.0f);
      }
#pragma unroll
      for (int c = 0; c < V; ++c) {
        keep_packed(xp[r][c]);
        if constexpr (ADD)
          row_store<T, E, true, FAST>(h + (row0 + r) * (int64_t)N - hd, (c * G + ls) * E, nw, ok[r],
                                      xp[r][c], hd);
        if constexpr (kHold && !kWideWeights) {
          keep_packed(gp[c]);
          if constexpr (!RMS) keep_packed(bp[c]);
        }
        Pack<WT, E> gl, bl;
        if constexpr (!kHold) {
          gl = gahead;
          if constexpr (!RMS) bl = bahead;
          if (c + 1 < V) {
            gahead = lookup(gamma, c + 1, 1.0f);
            if constexpr (!RMS) bahead = lookup(beta, c + 1, 0.0f);
          }
          __builtin_amdgcn_sched_barrier(0);
        }
        const Pack<WT, E>& gc = kHold ? gp[kHold ? c : 0] : gl;
        const Pack<WT, E>& bc = RMS ? gc : (kHold ? bp[kHold && !RMS ? c : 0] : bl);
        Pack<TY, E> o;
#pragma unroll
        for (int i = 0; i < E; ++i) {
          float v;
          if constexpr (RMS)
            v = (xp[r][c].get(i) * rs[r]) * gc.get(i);
          else if constexpr (sizeof(T) == 2)
            // (x - mean0) * rs - m1 * rs in one FMA: one instruction fewer an element;
            // on a constant row x - mean0 and m1 are exactly zero, so y is still beta
            v = fmaf(xp[r][c].get(i) - mean0[r], rs[r], nm1rs[r]) * gc.get(i) + bc.get(i);
          else
            v = (((xp[r][c].get(i) - mean0[r]) - m1[r]) * rs[r]) * gc.get(i) + bc.get(i);
          o.set(i, v);
        }
        row_store<TY, E, true, FAST>(yr, (c * G + ls) * E, nw, ok[r], o, hd);
        if constexpr (!kHold) __builtin_amdgcn_sched_barrier(0);
      }
      if (ok[r] && lane0 == 0) {
        if constexpr (!RMS)
          // (a row with an inf element has NaN variance; its mean is NaN as well, as the
          // Welford recurrence of the CPU kernel gives)
          if (mean) mean[row0 + r] = rs[r] == rs[r] ? mean0[r] + m1[r] : rs[r];
        if (rstd) rstd[row0 + r] = rs[r];
      }
    }
  }
}

// ---------------------------------------------------------------------------
// The same forward for 16-bit rows that fill a two-pack layout of whole wavefronts
// exactly (N == G * 2 * E, every row slot of every row block holds a row, no
// residual add, y in the row dtype): no access is conditional and no fill value is
// selected, the row index is wavefront-uniform, so the row pointers are scalar
// arithmetic and a lane adds one constant 32-bit offset.  One resident grid whose
// workgroups keep gamma / beta across their rows.  Arithmetic and results are
// those of norm_fwd_resident_kernel for the same layout, bit for bit.  Measured on
// one MI355X, bf16 rows x 16384 (LayerNorm / RMSNorm, us): N = 4096 45.8 / 43.8 ->
// 44.1 / 43.7 (fp32 weights 46.2 / 44.4 -> 45.5 / 43.6), 5120 (320 lanes) 58.2 /
// 55.2 -> 55.6 / 54.2; no gain at 8192, and requesting the next row ahead of the
// current one (as the backward does) measured slower here at every depth.
template <class T, class WT, int G, int BLOCK, bool RMS>
__global__ void __launch_bounds__(BLOCK)
norm_fwd_exact_kernel(const T* __restrict__ x, const WT* __restrict__ gamma,
                      const WT* __restrict__ beta, T* __restrict__ y, float* __restrict__ mean,
                      float* __restrict__ rstd, int64_t M, int N, float eps) {
  constexpr int E = elems_per_pack<T>::value;
  constexpr int V = 2;
  constexpr int RPB = BLOCK / G;
  static_assert(sizeof(T) == 2 && G % 64 == 0 && BLOCK % G == 0, "16-bit rows on whole wavefronts");
  __shared__ float red[reduce_lds_floats<G, BLOCK, 2>::value];
  int phase = 0;
  const int slot = threadIdx.x / G;
  const int lane0 = threadIdx.x % G;
  const float fN = (float)N;
  const float inv_n = 1.0f / fN;
  const int slot_u = __builtin_amdgcn_readfirstlane(slot);
  uint32_t voff[V];
  Pack<WT, E> gp[V], bp[RMS ? 1 : V];
#pragma unroll
  for (int c = 0; c < V; ++c) {
    const int e0 = (c * G + lane0) * E;
    voff[c] = (uint32_t)(e0 * (int)sizeof(T));
    gp[c] = gamma ? Pack<WT, E>::load(gamma + e0) : Pack<WT, E>::splat(1.0f);
    if constexpr (!RMS) bp[c] = beta ? Pack<WT, E>::load(beta + e0) : Pack<WT, E>::zero();
  }
  auto at = [](const T* rowp, uint32_t off) {
    return reinterpret_cast<const T*>(reinterpret_cast<const char*>(rowp) + off);
  };
  const int64_t nrb = M / RPB;
  for (int64_t rb = blockIdx.x; rb < nrb; rb += gridDim.x) {
    const int64_t row = rb * RPB + slot_u;
    const T* xr = x + row * (int64_t)N;
    Pack<T, E> xp[V];
#pragma unroll
    for (int c = 0; c < V; ++c) xp[c] = Pack<T, E>::load_stream(at(xr, voff[c]));
    float mean0 = 0.0f, m1 = 0.0f, rs;
    if constexpr (RMS) {
      float acc[1] = {0.0f};
#pragma unroll
      for (int c = 0; c < V; ++c)
#pragma unroll
        for (int i = 0; i < E; ++i) {
          const float v = xp[c].get(i);
          acc[0] = fmaf(v, v, acc[0]);
        }
      group_allreduce<G, BLOCK, 1, SumOp>(acc, red, phase);
      rs = row_rstd_of<T>(row_mean_of<T>(acc[0], fN, inv_n) + eps);
    } else {
      // the centre: the median of the row's first three elements (see the kernel above)
      const Pack<T, E> head = Pack<T, E>::load(xr);
      const float a = head.get(0), b = head.get(1), c3 = head.get(2);
      const float k = fmaxf(fminf(a, b), fminf(fmaxf(a, b), c3));
      mean0 = k;
      float acc[2] = {0.0f, 0.0f};
#pragma unroll
      for (int c = 0; c < V; ++c)
#pragma unroll
        for (int i = 0; i < E; ++i) {
          const float d = xp[c].get(i) - k;
          acc[0] += d;
          acc[1] = fmaf(d, d, acc[1]);
        }
      group_allreduce<G, BLOCK, 2, SumOp>(acc, red, phase);
      m1 = row_mean_of<T>(acc[0], fN, inv_n);
      float var = row_mean_of<T>(acc[1] - acc[0] * m1, fN, inv_n);
      var = var < 0.0f ? 0.0f : var;  // a select: a NaN row keeps NaN statistics
      rs = row_rstd_of<T>(var + eps);
    }
    const float nm1rs = -m1 * rs;
    T* yr = y + row * (int64_t)N;
#pragma unroll
    for (int c = 0; c < V; ++c) {
      keep_packed(xp[c]);
      Pack<T, E> o;
#pragma unroll
      for (int i = 0; i < E; ++i) {
        float v;
        if constexpr (RMS)
          v = (xp[c].get(i) * rs) * gp[c].get(i);
        else
          v = fmaf(xp[c].get(i) - mean0, rs, nm1rs) * gp[c].get(i) + bp[c].get(i);
        o.set(i, v);
      }
      o.store_stream(const_cast<T*>(at(yr, voff[c])));
    }
    if (lane0 == 0) {
      if constexpr (!RMS)
        if (mean) mean[row] = rs == rs ? mean0 + m1 : rs;
      if (rstd) rstd[row] = rs;
    }
  }
}

// The centre the long-row kernels shift their sums by: the median of the row's
// first three elements, the same value in every workgroup that works on the row.
// With a residual row `rr` (may be null) the row is h = x + res rounded to T.
template <class T>
__device__ __forceinline__ float split_row_centre(const T* xr, const T* rr, int N) {
  const int i1 = N > 1 ? 1 : 0, i2 = N > 2 ? 2 : 0;
  float a = (float)xr[0], b = (float)xr[i1], c = (float)xr[i2];
  if (rr != nullptr) {
    a = (float)(T)(a + (float)rr[0]);
    b = (float)(T)(b + (float)rr[i1]);
    c = (float)(T)(c + (float)rr[i2]);
  }
  return fmaxf(fminf(a, b), fminf(fmaxf(a, b), c));
}

// Packs a lane of the long-row kernels requests before it uses the first.
constexpr int kLongRowUnroll = 4;

// What a lane of the long-row forward holds of one pack between request and use.
template <class T, class WT, int E>
struct LongRowIn {
  Pack<T, E> x, r;   // the row and the residual row (r only with a residual)
  Pack<WT, E> g, b;  // gamma, beta (output pass only)
};

// x, or x + res formed in float32 and rounded once to T.
template <class T, int E, bool HASRES>
__device__ __forceinline__ Pack<T, E> sum_pack_of(const Pack<T, E>& x, const Pack<T, E>& r) {
  if constexpr (!HASRES) return x;
  Pack<T, E> p;
#pragma unroll
  for (int i = 0; i < E; ++i) p.set(i, x.get(i) + r.get(i));
  return p;
}

// Adds sum(x - k) and sum((x - k)^2) of one pack (its first `nvalid` elements when
// !WHOLE) to the float64 sums.  float32 rows: every term in float64, where the
// differences are exact.  16-bit rows: x - k is exact in float32 already (unless
// |k| is 2^16 times |x|), and the terms of a pack are added in float32 before they
// join the float64 sums: a quarter of the float64 instructions (they made the
// sums pass arithmetic-bound), and the rounding of a pack's sums -- 2^-24
// relative, independent from pack to pack -- stays orders below the 16-bit
// tolerance even when k lies a thousand standard deviations from the row.
template <class T, int E, bool RMS, bool WHOLE>
__device__ __forceinline__ void add_centred_sums(const Pack<T, E>& p, int nvalid, float kf,
                                                 double kd, double& s1, double& s2) {
  if constexpr (sizeof(T) == 2) {
    float t1 = 0.0f, t2 = 0.0f;
#pragma unroll
    for (int i = 0; i < E; ++i) {
      float d = p.get(i) - kf;
      if constexpr (!WHOLE) d = (i < nvalid) ? d : 0.0f;
      if constexpr (!RMS) t1 += d;
      t2 = fmaf(d, d, t2);
    }
    if constexpr (!RMS) s1 += (double)t1;
    s2 += (double)t2;
  } else {
#pragma unroll
    for (int i = 0; i < E; ++i) {
      double d = (double)p.get(i) - kd;
      if constexpr (!WHOLE) d = (i < nvalid) ? d : 0.0;
      if constexpr (!RMS) s1 += d;
      s2 = fma(d, d, s2);
    }
  }
}

// sum(x - k), sum((x - k)^2) over the packs [p0, p1) of a thread (see for_packs).
template <class T, int E, int BLOCK, bool RMS, bool HASRES>
__device__ __forceinline__ void long_row_sums(const T* xr, const T* rr, int N, int64_t p0,
                                              int64_t p1, float kf, double& s1, double& s2) {
  const double kd = (double)kf;
  for_packs<kLongRowUnroll, BLOCK>(
      p0, p1, (int64_t)(N / E),
      [&](int64_t pk, auto whole) {
        constexpr bool W = decltype(whole)::value;
        LongRowIn<T, T, E> d;
        d.x = load_pack_of<T, E, false, W>(xr, pk * E, N, 0.0f);
        if constexpr (HASRES) d.r = load_pack_of<T, E, false, W>(rr, pk * E, N, 0.0f);
        return d;
      },
      [&](int64_t pk, const LongRowIn<T, T, E>& d, auto whole) {
        constexpr bool W = decltype(whole)::value;
        add_centred_sums<T, E, RMS, W>(sum_pack_of<T, E, HASRES>(d.x, d.r), N - (int)(pk * E), kf,
                                       kd, s1, s2);
      });
}

// y = gamma * ((x - hi) - lo) * rs + beta (RMSNorm: gamma * x * rs) over the packs
// [p0, p1) of a thread; with a residual row the normalized row is h = x + res,
// written out as well.
template <class T, class WT, class TY, int E, int BLOCK, bool RMS, bool HASRES>
__device__ __forceinline__ void long_row_apply(const T* xr, const T* rr, const WT* gamma,
                                               const WT* beta, T* hr, TY* yr, int N, int64_t p0,
                                               int64_t p1, float hi, float lo, float rs) {
  const bool hg = gamma != nullptr, hb = !RMS && beta != nullptr;  // uniform over the launch
  for_packs<kLongRowUnroll, BLOCK>(
      p0, p1, (int64_t)(N / E),
      [&](int64_t pk, auto whole) {
        constexpr bool W = decltype(whole)::value;
        LongRowIn<T, WT, E> d;
        d.x = load_pack_of<T, E, true, W>(xr, pk * E, N, 0.0f);
        if constexpr (HASRES) d.r = load_pack_of<T, E, true, W>(rr, pk * E, N, 0.0f);
        d.g = hg ? load_pack_of<WT, E, false, W>(gamma, pk * E, N, 1.0f) : Pack<WT, E>::splat(1.0f);
        d.b = hb ? load_pack_of<WT, E, false, W>(beta, pk * E, N, 0.0f) : Pack<WT, E>::zero();
        return d;
      },
      [&](int64_t pk, const LongRowIn<T, WT, E>& d, auto whole) {
        constexpr bool W = decltype(whole)::value;
        const Pack<T, E> p = sum_pack_of<T, E, HASRES>(d.x, d.r);
        if constexpr (HASRES) store_pack_of<T, E, true, W>(hr, pk * E, N, p);
        Pack<TY, E> o;
#pragma unroll
        for (int i = 0; i < E; ++i) {
          float v;
          if constexpr (RMS)
            v = (p.get(i) * rs) * d.g.get(i);
          else
            v = (((p.get(i) - hi) - lo) * rs) * d.g.get(i) + d.b.get(i);
          o.set(i, v);
        }
        store_pack_of<TY, E, true, W>(yr, pk * E, N, o);
      });
}

// ---------------------------------------------------------------------------
// Forward for short ragged rows (N % E != 0, up to 64 lanes x kFlatMaxPacks packs) through
// LDS, as the softmax kernels for such rows (device/flat_rows.hpp): a run of
// `chunk_rows` consecutive rows, a multiple of 8, is one contiguous piece of X that
// starts and ends on a 16-byte boundary, so it enters and leaves LDS with whole aligned
// 128-bit accesses and HBM sees the pattern of a copy; a group of G lanes (inside one
// wavefront) then normalizes a row in place in LDS, VP packs a lane, read at the row's
// own alignment.  A lane owns the same columns in every row, so its gamma / beta packs
// are loaded once a workgroup.  Statistics: the centred sums of the register-resident
// kernel, reduced inside the wavefront.  Needs 16-byte aligned X and Y; the general
// kernels serve the rest.  Measured on MI355X against the general register-resident
// kernel, bf16, 131072 rows, LayerNorm / RMSNorm us: N = 17 15.7 / 10.0 -> 7.9 / 6.7, 100:
// 24.2 / 21.5 -> 15.1 / 12.8, 127: 32.6 / 29.9 -> 17.1 / 15.3, 257: 50.3 / 33.6 -> 41.2 / 32.0,
// 777: 99.3 / 81.1 -> 85.5 / 72.2, 1001: 112.5 / 97.4 -> 96.1 / 90.1, 2047: 219 / 197 -> 191 / 184.
template <class T, class WT, int G, int VP, int BLOCK, int LDSB, bool RMS>
__global__ void __launch_bounds__(BLOCK)
norm_fwd_flat_kernel(const T* __restrict__ x, const WT* __restrict__ gamma,
                     const WT* __restrict__ beta, T* __restrict__ y, float* __restrict__ mean,
                     float* __restrict__ rstd, int64_t M, int N, int chunk_rows, float eps) {
  constexpr int E = elems_per_pack<T>::value;
  constexpr int RPB = BLOCK / G;
  constexpr int U = LDSB / (BLOCK * 16);
  __shared__ __attribute__((aligned(16))) T buf[LDSB / sizeof(T) + E];
  const int64_t row0 = (int64_t)blockIdx.x * chunk_rows;
  const int rows_here = M - row0 < chunk_rows ? (int)(M - row0) : chunk_rows;
  const int nelem = rows_here * N;
  const int lane = threadIdx.x % G;
  // this lane's columns: the same in every row
  Pack<WT, E> gp[VP], bp[RMS ? 1 : VP];
#pragma unroll
  for (int c = 0; c < VP; ++c) {
    const int j = (c * G + lane) * E;
    gp[c] = gamma ? load_row_pack<WT, E, false>(gamma, j, N, true, 1.0f) : Pack<WT, E>::splat(1.0f);
    if constexpr (!RMS)
      bp[c] = beta ? load_row_pack<WT, E, false>(beta, j, N, true, 0.0f) : Pack<WT, E>::zero();
  }
  flat_stage_in<T, BLOCK, U>(x + row0 * (int64_t)N, buf, nelem);
  __syncthreads();
  const float fN = (float)N, inv_n = 1.0f / fN;
  for (int r = threadIdx.x / G; r < rows_here; r += RPB) {
    T* rowb = buf + r * N;
    float v[VP][E];
    float s = 0.0f;
#pragma unroll
    for (int c = 0; c < VP; ++c) {
      const int j = (c * G + lane) * E;
      Pack<T, E> p = Pack<T, E>::zero();
      if (j < N) p = flat_row_pack<T, E>(rowb, j);
#pragma unroll
      for (int i = 0; i < E; ++i) {
        v[c][i] = j + i < N ? p.get(i) : 0.0f;
        s += RMS ? v[c][i] * v[c][i] : v[c][i];
      }
    }
    // LayerNorm statistics as in the register-resident kernel: sums of x - k and
    // (x - k)^2 about a centre k -- for 16-bit rows the median of the row's first three
    // elements (one reduction round), for fp32 rows the rounded mean (a round of its
    // own) -- so that a constant row gives mean = the constant, zero variance and
    // y = beta bit for bit.
    float k = 0.0f, m1 = 0.0f, rs;
    if constexpr (RMS) {
      s = wave_group_allreduce<G, SumOp>(s);
      rs = row_rstd_of<T>(row_mean_of<T>(s, fN, inv_n) + eps);
    } else {
      if constexpr (sizeof(T) == 2) {
        const float a = (float)rowb[0], b = (float)rowb[N > 1 ? 1 : 0],
                    c3 = (float)rowb[N > 2 ? 2 : 0];
        k = fmaxf(fminf(a, b), fminf(fmaxf(a, b), c3));
      } else {
        s = wave_group_allreduce<G, SumOp>(s);
        k = s / fN;
      }
      float s1 = 0.0f, s2 = 0.0f;
#pragma unroll
      for (int c = 0; c < VP; ++c) {
        const int j = (c * G + lane) * E;
#pragma unroll
        for (int i = 0; i < E; ++i) {
          const float d = j + i < N ? v[c][i] - k : 0.0f;
          s1 += d;
          s2 = fmaf(d, d, s2);
        }
      }
      s1 = wave_group_allreduce<G, SumOp>(s1);
      s2 = wave_group_allreduce<G, SumOp>(s2);
      m1 = row_mean_of<T>(s1, fN, inv_n);
      float var = row_mean_of<T>(s2 - s1 * m1, fN, inv_n);
      var = var < 0.0f ? 0.0f : var;  // a select: a NaN row keeps NaN statistics
      rs = row_rstd_of<T>(var + eps);
    }
    const float nm1rs = -m1 * rs;
#pragma unroll
    for (int c = 0; c < VP; ++c) {
      const int j = (c * G + lane) * E;
      Pack<T, E> o;
#pragma unroll
      for (int i = 0; i < E; ++i) {
        if constexpr (RMS)
          o.set(i, (v[c][i] * rs) * gp[c].get(i));
        else if constexpr (sizeof(T) == 2)
          o.set(i, fmaf(v[c][i] - k, rs, nm1rs) * gp[c].get(i) + bp[c].get(i));
        else
          o.set(i, (((v[c][i] - k) - m1) * rs) * gp[c].get(i) + bp[c].get(i));
      }
      if (j < N) flat_row_store<T, E>(rowb, j, N - j, o);
    }
    if (lane == 0) {
      if constexpr (!RMS)
        if (mean) mean[row0 + r] = rs == rs ? k + m1 : rs;  // NaN variance: NaN mean
      if (rstd) rstd[row0 + r] = rs;
    }
  }
  __syncthreads();
  flat_stage_out<T, BLOCK, U>(y + row0 * (int64_t)N, buf, nelem);
}

// ---------------------------------------------------------------------------
// Backward for the rows norm_fwd_flat_kernel serves (short ragged rows, 16-byte aligned
// dY, X and dX): pieces of `chunk_rows` consecutive rows of dY and X enter LDS with
// whole aligned accesses, a group of G lanes works a row there (s1, s2 reduced inside
// the wavefront, dX written over the row of dY in LDS), and the piece of dX leaves with
// whole 128-bit stores.  A lane owns the same columns in every row, so it keeps their
// dgamma / dbeta sums in registers over all the pieces its workgroup walks (a grid-stride
// loop over pieces, so the partial rows are as many as the general kernel's).  At the
// end the lane groups of the workgroup are folded through LDS in a fixed order and one
// fp32 row goes to the [gridDim.x, N] partial buffers; colsum_finalize_kernel adds those.
// Arithmetic of a row: that of norm_bwd_resident_kernel.
template <class T, class WT, int G, int VP, int BLOCK, int LDSB, bool RMS>
__global__ void __launch_bounds__(BLOCK)
norm_bwd_flat_kernel(const T* __restrict__ dy, const T* __restrict__ x,
                     const float* __restrict__ mean, const float* __restrict__ rstd,
                     const WT* __restrict__ gamma, T* __restrict__ dx,
                     float* __restrict__ part_dg, float* __restrict__ part_db, int64_t M, int N,
                     int chunk_rows) {
  constexpr int E = elems_per_pack<T>::value;
  constexpr int RPB = BLOCK / G;
  constexpr int U = LDSB / (BLOCK * 16);
  // two tensors of a piece; afterwards the fold of the column sums (RPB * G * VP * E floats)
  constexpr int kBufElems = LDSB / (int)sizeof(T) + E;
  constexpr int kFoldBytes = BLOCK * VP * E * (int)sizeof(float);
  constexpr int kBytes = 2 * kBufElems * (int)sizeof(T) > kFoldBytes
                             ? 2 * kBufElems * (int)sizeof(T) : kFoldBytes;
  __shared__ __attribute__((aligned(16))) unsigned char lds[kBytes];
  T* bd = reinterpret_cast<T*>(lds);
  T* bx = bd + kBufElems;
  const int lane = threadIdx.x % G;
  const int slot = threadIdx.x / G;
  const bool want_cols = part_dg != nullptr;  // uniform
  const float fN = (float)N, inv_n = 1.0f / fN;
  Pack<WT, E> gp[VP];
  float dg[VP][E], db[RMS ? 1 : VP][RMS ? 1 : E];
#pragma unroll
  for (int c = 0; c < VP; ++c) {
    const int j = (c * G + lane) * E;
    gp[c] = gamma ? load_row_pack<WT, E, false>(gamma, j, N, true, 1.0f) : Pack<WT, E>::splat(1.0f);
#pragma unroll
    for (int i = 0; i < E; ++i) {
      dg[c][i] = 0.0f;
      if constexpr (!RMS) db[c][i] = 0.0f;
    }
  }
  const int64_t npieces = (M + chunk_rows - 1) / chunk_rows;
  for (int64_t piece = blockIdx.x; piece < npieces; piece += gridDim.x) {
    const int64_t row0 = piece * chunk_rows;
    const int rows_here = M - row0 < chunk_rows ? (int)(M - row0) : chunk_rows;
    const int nelem = rows_here * N;
    flat_stage_in2<T, BLOCK, U>(dy + row0 * (int64_t)N, bd, x + row0 * (int64_t)N, bx, nelem);
    __syncthreads();
    for (int r = slot; r < rows_here; r += RPB) {
      T* rd = bd + r * N;
      const T* rx = bx + r * N;
      const float mu = RMS ? 0.0f : mean[row0 + r];
      const float rs = rstd[row0 + r];
      float gy[VP][E], xh[VP][E];
      float s1 = 0.0f, s2 = 0.0f;
#pragma unroll
      for (int c = 0; c < VP; ++c) {
        const int j = (c * G + lane) * E;
        Pack<T, E> pd = Pack<T, E>::zero(), px = Pack<T, E>::zero();
        if (j < N) {
          pd = flat_row_pack<T, E>(rd, j);
          px = flat_row_pack<T, E>(rx, j);
        }
#pragma unroll
        for (int i = 0; i < E; ++i) {
          const bool in = j + i < N;
          gy[c][i] = in ? pd.get(i) : 0.0f;
          xh[c][i] = in ? (px.get(i) - mu) * rs : 0.0f;
          const float g = gy[c][i] * gp[c].get(i);
          if constexpr (!RMS) s1 += g;
          s2 = fmaf(g, xh[c][i], s2);
          dg[c][i] = fmaf(gy[c][i], xh[c][i], dg[c][i]);
          if constexpr (!RMS) db[c][i] += gy[c][i];
        }
      }
      if constexpr (!RMS) s1 = wave_group_allreduce<G, SumOp>(s1);
      s2 = wave_group_allreduce<G, SumOp>(s2);
      const float term1 = row_mean_of<T>(rs, fN, inv_n);
#pragma unroll
      for (int c = 0; c < VP; ++c) {
        const int j = (c * G + lane) * E;
        Pack<T, E> o;
#pragma unroll
        for (int i = 0; i < E; ++i) {
          // dx = (rs / N) * (N * g - xhat * s2 - s1), g = dy * gamma
          float f = fN * (gy[c][i] * gp[c].get(i));
          f -= xh[c][i] * s2;
          if constexpr (!RMS) f -= s1;
          o.set(i, f * term1);
        }
        if (j < N) flat_row_store<T, E>(rd, j, N - j, o);
      }
    }
    __syncthreads();
    if (dx != nullptr) flat_stage_out<T, BLOCK, U>(dx + row0 * (int64_t)N, bd, nelem);
    __syncthreads();  // the buffers are filled again, or folded over, next
  }
  if (!want_cols) return;
  // fold the lane groups that own the same columns, in slot order, one sum kind at a time
  float* fold = reinterpret_cast<float*>(lds);
  float* out_g = part_dg + (int64_t)blockIdx.x * N;
  float* out_b = RMS ? nullptr : part_db + (int64_t)blockIdx.x * N;
  constexpr int NPASS = RMS ? 1 : 2;
  constexpr int COLS = G * VP * E;  // columns a lane group covers
#pragma unroll
  for (int pass = 0; pass < NPASS; ++pass) {
#pragma unroll
    for (int c = 0; c < VP; ++c)
#pragma unroll
      for (int i = 0; i < E; ++i)
        fold[slot * COLS + (c * G + lane) * E + i] =
            pass == 0 ? dg[c][i] : db[RMS ? 0 : c][RMS ? 0 : i];
    __syncthreads();
    for (int j = threadIdx.x; j < N; j += BLOCK) {
      float t = 0.0f;
      for (int sl = 0; sl < RPB; ++sl) t += fold[sl * COLS + j];
      (pass == 0 ? out_g : out_b)[j] = t;
    }
    __syncthreads();
  }
}

// ---------------------------------------------------------------------------
// Forward for rows too wide to hold in registers: one workgroup per row, the
// row is streamed from memory twice (statistics, normalize); the second pass
// hits L2 / Infinity Cache for any realistic row.  LayerNorm sums (x - k) and
// (x - k)^2 in float64, k = the median of the row's first three elements (see
// the split-row kernels below for why float64); RMSNorm sums x^2 in float32,
// where nothing cancels.
// res / h (null, or both given): the row is h = x + res, written out in the
// second pass (see the resident kernel); TY: the element type of y.
template <class T, class WT, int BLOCK, bool RMS, class TY = T>
__global__ void __launch_bounds__(BLOCK)
norm_fwd_stream_kernel(const T* __restrict__ x, const T* res, const WT* __restrict__ gamma,
                       const WT* __restrict__ beta, T* h, TY* __restrict__ y,
                       float* __restrict__ mean, float* __restrict__ rstd, int64_t M, int N,
                       float eps) {
  constexpr int E = elems_per_pack<T>::value;
  __shared__ float red[reduce_lds_floats<BLOCK, BLOCK, 2>::value];
  __shared__ double red64[RMS ? 1 : 2 * (BLOCK / 64)];
  __shared__ float stat[3];
  int phase = 0;
  const float fN = (float)N;
  const int npacks = (N + E - 1) / E;
  for (int64_t row = blockIdx.x; row < M; row += gridDim.x) {
    const T* xr = x + row * (int64_t)N;
    const T* rr = res ? res + row * (int64_t)N : nullptr;
    TY* yr = y + row * (int64_t)N;
    // mean = hi + lo: the saved statistic and the remainder of the float64 mean, kept
    // apart so that the rounding of the saved mean never enters y
    float hi = 0.0f, lo = 0.0f, rs;
    if constexpr (RMS) {
      // (float64 partial sums of float32 pack sums: see add_centred_sums)
      double s1 = 0.0, s2 = 0.0;
      if (rr != nullptr)
        long_row_sums<T, E, BLOCK, true, true>(xr, rr, N, 0, npacks, 0.0f, s1, s2);
      else
        long_row_sums<T, E, BLOCK, true, false>(xr, rr, N, 0, npacks, 0.0f, s1, s2);
      float acc[1] = {(float)s2};
      group_allreduce<BLOCK, BLOCK, 1, SumOp>(acc, red, phase);
      rs = 1.0f / sqrtf(acc[0] / fN + eps);  // once a row of >= 32 Ki elements: exact
    } else {
      const float kf = split_row_centre(xr, rr, N);
      const double k = (double)kf;
      double s1 = 0.0, s2 = 0.0;
      if (rr != nullptr)
        long_row_sums<T, E, BLOCK, false, true>(xr, rr, N, 0, npacks, kf, s1, s2);
      else
        long_row_sums<T, E, BLOCK, false, false>(xr, rr, N, 0, npacks, kf, s1, s2);
      block_sum2_f64<BLOCK>(s1, s2, red64);
      if (threadIdx.x == 0) {
        const double dN = (double)N;
        const double m1 = s1 / dN;
        const double mu = k + m1;
        double var = (s2 - s1 * m1) / dN;
        var = var < 0.0 ? 0.0 : var;  // a select: a NaN row keeps NaN statistics
        stat[0] = (float)mu;
        stat[1] = (float)(mu - (double)stat[0]);
        stat[2] = (float)(1.0 / sqrt(var + (double)eps));
      }
      __syncthreads();
      hi = stat[0];
      lo = stat[1];
      rs = stat[2];
    }
    // (h may lie on top of x or res: the block reduction above is a barrier, so every
    // thread has finished the first pass before any of h is written; a thread then
    // reads and writes the same elements)
    T* hr = rr != nullptr ? h + row * (int64_t)N : nullptr;
    if (rr != nullptr)
      long_row_apply<T, WT, TY, E, BLOCK, RMS, true>(xr, rr, gamma, beta, hr, yr, N, 0, npacks, hi,
                                                     lo, rs);
    else
      long_row_apply<T, WT, TY, E, BLOCK, RMS, false>(xr, rr, gamma, beta, hr, yr, N, 0, npacks,
                                                      hi, lo, rs);
    if (threadIdx.x == 0) {
      if constexpr (!RMS)
        if (mean) mean[row] = rs == rs ? hi : rs;  // NaN variance: NaN mean
      if (rstd) rstd[row] = rs;
    }
    // stat[] is rewritten for the next row only after every thread has passed the
    // barrier inside the next block sum, i.e. after it has read this row's values
  }
}

// ---------------------------------------------------------------------------
// Forward for rows beyond the registers of one workgroup, in ONE pass over X: a
// row is held in the registers of a team of workgroups.  The grid is at most two
// workgroups of 512 threads a compute unit, all resident at once; workgroup b
// belongs to team b / team and keeps chunk b % team of the team's current row: V
// packs a lane, V * 512 packs a workgroup (up to 16: 128 KiB a workgroup, 64 MiB on
// 256 compute units; the last chunk of a row may hold fewer).  It sums its chunk
// (float64 sums about the row's centre, as the split-row kernels below), publishes
// the two partial sums in its entry of library-owned device memory and waits until
// every workgroup of its team has; each then adds the team's partial sums in chunk
// order (the same statistics in every workgroup, run to run), normalizes its chunk
// out of its registers and writes Y.  X is read once and Y written once, where the
// split-row kernels read X twice (they remain for the calls this kernel does not
// serve: a residual add, a cast, ragged rows, Y on top of X, a stream under
// capture).  Role in the reference: the split-row regime of Norm.h:632-812, whose
// partial results also cross work-groups through global memory, between two
// launches.
//
// A full chunk runs straight-line code: V unconditional loads in flight a lane,
// and on the way out the weights of the next kTeamGroup packs are requested before
// the current ones are normalized and stored, so no pack waits for the store of the
// pack before it (bf16 [512, 401408]: 177 -> 170 us).
//
// What crosses workgroups and how the wait is bounded: device/team.hpp.  A workgroup
// that stops waiting without its team sums the whole row itself -- a second pass over X,
// whose statistics agree with the team's to rounding -- loads its chunk again and goes
// on.  Every wave reaches the end of the kernel whatever the other workgroups do, and
// every row is written.
//
// GROUP: the rows are the (sample, group) slabs of a GroupNorm whose channels are whole
// packs (`group.packs_per_channel` packs each): gamma and beta hold one value a channel,
// looked up by the pack's position in the row, and mean / rstd leave in the weight
// dtype ST, as native_group_norm returns them.  Everything else is the LayerNorm's.
struct TeamGroupShape {
  int groups = 1;             // groups a sample: row r belongs to group r % groups
  int channels = 1;           // channels a group
  int packs_per_channel = 1;  // HxW / E
};

template <class T, class WT, int V, bool RMS, bool GROUP = false, class ST = float>
__global__ void __launch_bounds__(kTeamBlock, kTeamPerCu * kTeamBlock / 256)
norm_fwd_team_kernel(const T* __restrict__ x, const WT* __restrict__ gamma,
                     const WT* __restrict__ beta, T* __restrict__ y, ST* __restrict__ mean,
                     ST* __restrict__ rstd, int64_t M, int N, float eps, int team,
                     int64_t chunk_packs, TeamSlot* slot, unsigned int call_id,
                     unsigned long long wait_ticks, TeamGroupShape group = TeamGroupShape{}) {
  static_assert(!(GROUP && RMS), "GroupNorm is a LayerNorm over a slab");
  constexpr int E = elems_per_pack<T>::value;
  constexpr int BLOCK = kTeamBlock;
  __shared__ double red[2 * (BLOCK / 64)];
  __shared__ double tpart[kTeamMaxWorkgroups][2];
  __shared__ float stat[4];
  const int tm = (int)blockIdx.x / team;
  const int c = (int)blockIdx.x - tm * team;
  const int teams = (int)gridDim.x / team;
  const int64_t npacks = (int64_t)N / E;
  const int64_t p0 = (int64_t)c * chunk_packs;
  const int64_t p1 = p0 + chunk_packs < npacks ? p0 + chunk_packs : npacks;
  const bool hg = gamma != nullptr, hb = !RMS && beta != nullptr;
  const double dN = (double)N;
  // Pack k of the lane lies k * BLOCK + threadIdx.x packs into the chunk: a scalar
  // pointer per pack and one 32-bit byte offset a lane (no 64-bit address a pack in
  // vector registers, which 16 packs a lane have no room for).
  const int nloc = p1 > p0 ? (int)(p1 - p0) : 0;  // packs of this chunk
  const bool full = nloc == V * BLOCK;  // (uniform) every lane holds V packs: all chunks but a row's last
  const int64_t pbase = nloc > 0 ? p0 : 0;
  const uint32_t loff = (uint32_t)(threadIdx.x * 16);
  // (the sum is formed as a pointer into global memory: a pointer made from an integer
  // is otherwise a generic one, and generic accesses wait for everything outstanding)
  auto at = [](auto* p, uint32_t off) {
    using Elem = std::remove_pointer_t<decltype(p)>;
    typedef __attribute__((address_space(1))) Elem* GlobalPtr;
    return (Elem*)reinterpret_cast<GlobalPtr>(reinterpret_cast<uintptr_t>(p) + off);
  };
  // mean = hi + lo and rstd of a row from its centred sums (see the split-row kernels)
  auto set_stats = [&](double t1, double t2, double kd) {
    if constexpr (RMS) {
      stat[0] = 0.0f;
      stat[1] = 0.0f;
      stat[2] = (float)(1.0 / sqrt(t2 / dN + (double)eps));
    } else {
      const double m1 = t1 / dN;
      const double mu = kd + m1;
      double var = (t2 - t1 * m1) / dN;
      var = var < 0.0 ? 0.0 : var;  // (a select: NaN stays NaN)
      const float hi = (float)mu;
      stat[0] = var == var ? hi : (float)var;  // NaN variance: NaN mean
      stat[1] = (float)(mu - (double)hi);
      stat[2] = (float)(1.0 / sqrt(var + (double)eps));
    }
  };
  unsigned int round = 0;
  for (int64_t row = tm; row < M; row += teams, ++round) {
    TeamEntry* entries = slot->entry[round & 1u];
    if (threadIdx.x == 0) team_store(&entries[blockIdx.x].tag, 0ull);
    const T* xr = x + row * (int64_t)N;
    const T* xb = xr + pbase * E;
    Pack<T, E> xp[V];
    if (full) {
      // (straight-line code: V requests in flight a lane, nothing conditional)
#pragma unroll
      for (int k = 0; k < V; ++k) xp[k] = Pack<T, E>::load_stream(at(xb + k * BLOCK * E, loff));
    } else {
#pragma unroll
      for (int k = 0; k < V; ++k) {
        xp[k] = Pack<T, E>::zero();
        if (k * BLOCK + (int)threadIdx.x < nloc)
          xp[k] = Pack<T, E>::load_stream(at(xb + k * BLOCK * E, loff));
      }
    }
    const float kf = RMS ? 0.0f : split_row_centre(xr, (const T*)nullptr, N);
    const double kd = (double)kf;
    double s1 = 0.0, s2 = 0.0;
#pragma unroll
    for (int k = 0; k < V; ++k) {
      keep_packed(xp[k]);
      if (full || k * BLOCK + (int)threadIdx.x < nloc)
        add_centred_sums<T, E, RMS, true>(xp[k], E, kf, kd, s1, s2);
    }
    block_sum2_f64<BLOCK>(s1, s2, red);
    if (threadIdx.x < 64) {  // the first wavefront publishes, waits and adds up
      const int lane = (int)threadIdx.x;
      const bool complete = team_publish_and_gather(slot, entries, tm, team, call_id, round,
                                                    wait_ticks, s1, s2, tpart);
      // (the lanes of a wavefront see one another's LDS stores in program order)
      if (lane == 0) {
        if (!complete) {
          stat[3] = 1.0f;
        } else {
          double t1 = 0.0, t2 = 0.0;
          for (int j = 0; j < team; ++j) {
            t1 += tpart[j][0];
            t2 += tpart[j][1];
          }
          set_stats(t1, t2, kd);
          stat[3] = 0.0f;
        }
      }
    }
    __syncthreads();
    if (stat[3] != 0.0f) {  // (uniform over the workgroup)
      // The team did not come together: this workgroup sums the whole row itself (the
      // row is X, which no workgroup writes), then takes its chunk again, whose
      // registers the pass over the row has used.
      double w1 = 0.0, w2 = 0.0;
      long_row_sums<T, E, BLOCK, RMS, false>(xr, (const T*)nullptr, N, 0, npacks, kf, w1, w2);
      block_sum2_f64<BLOCK>(w1, w2, red);
      if (threadIdx.x == 0) set_stats(w1, w2, kd);
      __syncthreads();
#pragma unroll
      for (int k = 0; k < V; ++k) {
        xp[k] = Pack<T, E>::zero();
        if (k * BLOCK + (int)threadIdx.x < nloc)
          xp[k] = Pack<T, E>::load_stream(at(xb + k * BLOCK * E, loff));
      }
    }
    const float hi = stat[0], lo = stat[1], rs = stat[2];
    T* yb = y + row * (int64_t)N + pbase * E;
    const WT* gb = (hg ? gamma : reinterpret_cast<const WT*>(x)) + pbase * E;
    const WT* bb = (hb ? beta : reinterpret_cast<const WT*>(x)) + pbase * E;
    // (opaque: the 2 * V weight addresses, the same for every row, would otherwise be
    // formed once ahead of the row loop and kept -- spilled -- across it)
    const uint32_t woff = (uint32_t)(lane_again((int)threadIdx.x) * E * (int)sizeof(WT));
    if constexpr (GROUP) {
      // one gamma and one beta a pack: those of the channel the pack lies in
      const int ch0 = (int)(row % group.groups) * group.channels;
      const uint32_t pk0 = (uint32_t)pbase + (uint32_t)lane_again((int)threadIdx.x);
      auto channel = [&](int k) {
        return ch0 + (int)((pk0 + (uint32_t)(k * BLOCK)) / (uint32_t)group.packs_per_channel);
      };
      auto normalized1 = [&](const Pack<T, E>& xk, float ga, float be) {
        Pack<T, E> o;
        const float gr = ga * rs;
#pragma unroll
        for (int i = 0; i < E; ++i) o.set(i, ((xk.get(i) - hi) - lo) * gr + be);
        return o;
      };
      if (full && hg && hb) {
        // (as below: the weights of the next packs are requested before these are stored)
        constexpr int GS = kTeamGroup, NG = (V + GS - 1) / GS;
        // (kept as loaded: widening a value waits for it, and that belongs to the turn
        // that uses it)
        WT wg[2][GS], wb[2][GS];
        auto request = [&](int g, int buf) {
#pragma unroll
          for (int u = 0; u < GS; ++u) {
            const int k = g * GS + u;
            if (k < V) {
              const int ch = channel(k);
              wg[buf][u] = gamma[ch];
              wb[buf][u] = beta[ch];
            }
          }
        };
        request(0, 0);
#pragma unroll
        for (int g = 0; g < NG; ++g) {
          if (g + 1 < NG) request(g + 1, (g + 1) & 1);
          __builtin_amdgcn_sched_barrier(0);
#pragma unroll
          for (int u = 0; u < GS; ++u) {
            const int k = g * GS + u;
            if (k < V) {
              keep_packed(xp[k]);
              normalized1(xp[k], (float)wg[g & 1][u], (float)wb[g & 1][u])
                  .store_stream(at(yb + k * BLOCK * E, loff));
            }
          }
          __builtin_amdgcn_sched_barrier(0);
        }
      } else {
#pragma unroll
        for (int k = 0; k < V; ++k) {
          if (k * BLOCK + (int)threadIdx.x < nloc) {
            keep_packed(xp[k]);
            const int ch = channel(k);
            const float ga = hg ? (float)gamma[ch] : 1.0f;
            const float be = hb ? (float)beta[ch] : 0.0f;
            normalized1(xp[k], ga, be).store_stream(at(yb + k * BLOCK * E, loff));
          }
        }
      }
      if (c == 0 && threadIdx.x == 0) {
        if (mean) mean[row] = (ST)hi;
        if (rstd) rstd[row] = (ST)rs;
      }
      continue;
    }
    auto normalized = [&](const Pack<T, E>& xk, const Pack<WT, E>& g, const Pack<WT, E>& b) {
      Pack<T, E> o;
#pragma unroll
      for (int i = 0; i < E; ++i) {
        float v;
        if constexpr (RMS)
          v = (xk.get(i) * rs) * g.get(i);
        else
          v = (((xk.get(i) - hi) - lo) * rs) * g.get(i) + b.get(i);
        o.set(i, v);
      }
      return o;
    };
    if (full && hg && (RMS || hb)) {
      // A full chunk with its weights: straight-line code in groups of kTeamGroup packs.
      // The weights of the next group are requested before the current group is worked
      // on and stored, so the wait for a group's weights never includes the stores of
      // the group before it (requests complete in order: behind a conditional store,
      // or a weight load issued after it, every pack would wait for the one before to
      // be written).
      // (as many packs' weights ahead as the registers beside the row allow: two, one,
      // or -- 16 packs a lane with float32 weights beside 16-bit rows -- none)
      constexpr int WP = (RMS ? 1 : 2) * (int)sizeof(WT) * E / 4;  // registers of a pack's weights
      constexpr int ROOM = 92 - 4 * V;
      constexpr int GS = ROOM >= 4 * WP ? kTeamGroup : 1, NG = (V + GS - 1) / GS;
      constexpr int NB = ROOM >= 2 * WP ? 2 : 1;
      Pack<WT, E> wg[NB][GS], wb[RMS ? 1 : NB][RMS ? 1 : GS];
      auto request = [&](int g, int buf) {
#pragma unroll
        for (int u = 0; u < GS; ++u) {
          const int k = g * GS + u;
          if (k < V) {
            wg[buf][u] = Pack<WT, E>::load(at(gb + k * BLOCK * E, woff));
            if constexpr (!RMS) wb[buf][u] = Pack<WT, E>::load(at(bb + k * BLOCK * E, woff));
          }
        }
      };
      if constexpr (NB == 2) request(0, 0);
#pragma unroll
      for (int g = 0; g < NG; ++g) {
        if constexpr (NB == 2) {
          if (g + 1 < NG) request(g + 1, (g + 1) & 1);
        } else {
          request(g, 0);
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int u = 0; u < GS; ++u) {
          const int k = g * GS + u;
          if (k < V) {
            keep_packed(xp[k]);
            const int buf = NB == 2 ? (g & 1) : 0;
            const Pack<T, E> o = normalized(xp[k], wg[buf][u], wb[RMS ? 0 : buf][RMS ? 0 : u]);
            o.store_stream(at(yb + k * BLOCK * E, loff));
          }
        }
        __builtin_amdgcn_sched_barrier(0);
      }
    } else {
#pragma unroll
    for (int k = 0; k < V; ++k) {
      if (k * BLOCK + (int)threadIdx.x < nloc) {
        keep_packed(xp[k]);
        const Pack<WT, E> g =
            hg ? Pack<WT, E>::load(at(gb + k * BLOCK * E, woff)) : Pack<WT, E>::splat(1.0f);
        const Pack<WT, E> b =
            hb ? Pack<WT, E>::load(at(bb + k * BLOCK * E, woff)) : Pack<WT, E>::zero();
        normalized(xp[k], g, b).store_stream(at(yb + k * BLOCK * E, loff));
      }
    }
    }
    if (c == 0 && threadIdx.x == 0) {
      if constexpr (!RMS)
        if (mean) mean[row] = (ST)hi;
      if (rstd) rstd[row] = (ST)rs;
    }
    // (stat[], tpart[] and red[] are rewritten for the next row only behind the barrier
    // inside the next block sum, which every thread reaches after it has read them)
  }
}

// ---------------------------------------------------------------------------
// The forward of such rows when a team has many of them to do: the team holds R rows at a
// time, workgroup c the packs [c * V * BLOCK, (c + 1) * V * BLOCK) of each (V packs a lane and
// row), so a lane meets the same columns in every row and keeps their gamma / beta in
// registers for the whole call (norm_fwd_team_kernel looks them up again for every row: at
// ten million elements a row that is as much traffic as X).  Three register sets: group j of
// a team lives in set j % 3; in round j a workgroup requests group j + 2, sums group j + 1
// (requested a round ago) and publishes its 2 R float64 sums, gathers group j (published a
// round earlier) and writes its Y: neither the loads nor the exchange are waited for with
// nothing else to do.  One workgroup a compute unit.  The statistics are those of norm_fwd_team_kernel (float64 sums about the median of
// the row's first three elements; mean = hi + lo).  A workgroup whose wait runs out sums its
// R rows itself (Y must not overlap X) and loads its packs again.
template <class T, class WT, bool RMS, int R, int V>
__global__ void __launch_bounds__(kTeamBlock, kTeamBlock / 256)
norm_fwd_rows_team_kernel(const T* __restrict__ x, const WT* __restrict__ gamma,
                          const WT* __restrict__ beta, T* __restrict__ y,
                          float* __restrict__ mean, float* __restrict__ rstd, int64_t M, int N,
                          float eps, int team, TeamSlot* slot, unsigned int call_id,
                          unsigned long long wait_ticks) {
  constexpr int E = elems_per_pack<T>::value;
  constexpr int BLOCK = kTeamBlock;
  constexpr int K = 2 * R;
  // (red, stat and failed by round parity: a round's values are read while the next round's
  // are already being written)
  __shared__ double red[2][(BLOCK / 64) * K];
  __shared__ float stat[2][R][3];  // a row's mean (hi, lo) and rstd
  __shared__ int failed[2];
  __shared__ int lost;  // the workgroup has stopped waiting for its team (see team_word_tag)
  if (threadIdx.x == 0) lost = 0;  // (read behind the barrier of the first sum at the earliest)
  // from five packs a lane on gamma lives in LDS (a pack a lane and k), not in registers
  constexpr bool GL = V > 4;
  __shared__ Pack<WT, E> gl[GL ? V : 1][GL ? BLOCK : 1];
  const int tm = (int)blockIdx.x / team;
  const int c = (int)blockIdx.x - tm * team;
  const int teams = (int)gridDim.x / team;
  const int npacks = N / E;
  const int pk0 = c * (V * BLOCK) + (int)threadIdx.x;
  const int64_t ngroups = (M + R - 1) / R;
  const double dN = (double)N;
  const bool hb = !RMS && beta != nullptr;
  Pack<WT, E> pg[GL ? 1 : V], pb[RMS ? 1 : V];
#pragma unroll
  for (int k = 0; k < V; ++k) {
    const bool held = pk0 + k * BLOCK < npacks;
    Pack<WT, E> gk = Pack<WT, E>::splat(1.0f);
    if (gamma != nullptr && held) gk = Pack<WT, E>::load(gamma + (int64_t)(pk0 + k * BLOCK) * E);
    if constexpr (GL)
      gl[k][threadIdx.x] = gk;  // (read back by the same lane only)
    else
      pg[k] = gk;
    if constexpr (!RMS) {
      pb[k] = Pack<WT, E>::zero();
      if (hb && held) pb[k] = Pack<WT, E>::load(beta + (int64_t)(pk0 + k * BLOCK) * E);
    }
  }
  const uint32_t loff = (uint32_t)(pk0 < npacks ? pk0 : 0) * 16u;
  auto at = [](auto* p, uint32_t off) {
    using Elem = std::remove_pointer_t<decltype(p)>;
    typedef __attribute__((address_space(1))) Elem* GlobalPtr;
    return (Elem*)reinterpret_cast<GlobalPtr>(reinterpret_cast<uintptr_t>(p) + off);
  };
  auto row_of = [&](int64_t g, int r) { return g * R + r < M ? g * R + r : M - 1; };
  // A register set: the lane's packs of the R rows of a group and the rows' first three
  // elements (the centre of a row's sums is their median: requested with the packs, so
  // that nothing waits for them later).
  struct Set {
    Pack<T, E> px[R * V];
    T head[R][3];
  };
  auto load_group = [&](int64_t g, Set& s) {
    const int i1 = N > 1 ? 1 : 0, i2 = N > 2 ? 2 : 0;
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const int64_t row = g * R + r;
      if constexpr (!RMS) {
        const T* xr = x + row_of(g, r) * (int64_t)N;
        s.head[r][0] = xr[0];
        s.head[r][1] = xr[i1];
        s.head[r][2] = xr[i2];
      }
#pragma unroll
      for (int k = 0; k < V; ++k) {
        s.px[r * V + k] = Pack<T, E>::zero();
        if (pk0 + k * BLOCK < npacks && row < M)
          s.px[r * V + k] = Pack<T, E>::load_stream(at(x + row * (int64_t)N + k * BLOCK * E, loff));
      }
    }
  };
  // (split_row_centre of the row, from the elements the set holds)
  auto centre = [&](const Set& s, int r) {
    if constexpr (RMS) return 0.0f;
    const float a = (float)s.head[r][0], b = (float)s.head[r][1], cc = (float)s.head[r][2];
    return fmaxf(fminf(a, b), fminf(fmaxf(a, b), cc));
  };
  // mean = hi + lo and rstd of a row from its centred sums (see the split-row kernels)
  auto set_stats = [&](int par, int r, double t1, double t2, double kd) {
    if constexpr (RMS) {
      stat[par][r][0] = 0.0f;
      stat[par][r][1] = 0.0f;
      stat[par][r][2] = (float)(1.0 / sqrt(t2 / dN + (double)eps));
    } else {
      const double m1 = t1 / dN;
      const double mu = kd + m1;
      double var = (t2 - t1 * m1) / dN;
      var = var < 0.0 ? 0.0 : var;  // (a select: NaN stays NaN)
      const float hi = (float)mu;
      stat[par][r][0] = var == var ? hi : (float)var;  // NaN variance: NaN mean
      stat[par][r][1] = (float)(mu - (double)hi);
      stat[par][r][2] = (float)(1.0 / sqrt(var + (double)eps));
    }
  };
  // First wavefront, at the start of a round: the sums of group g (in set s, published a
  // round ago) across the team and its statistics, for the threads behind the round's
  // barrier; then the wavefront's request of group g2 into s2 -- only now: the exchange
  // waits for everything the wavefront has outstanding, and a request made before it would
  // put the machine's whole burst of loads in its way.
  auto gather = [&](int64_t g, unsigned int round, const Set& s, int64_t g2, Set& s2) {
    const int par = (int)(round & 1u);
    double tot[K];
    const bool complete =
        team_gather_sums_f64<K>(slot, slot->entry[round & 3u] + tm * team, team, call_id, round,
                                wait_ticks, tot);
    if (threadIdx.x == 0) {
      failed[par] = complete ? 0 : 1;
      if (!complete) lost = 1;
      if (complete) {
#pragma unroll
        for (int r = 0; r < R; ++r) set_stats(par, r, tot[2 * r], tot[2 * r + 1], (double)centre(s, r));
      }
    }
    if (g2 >= 0) load_group(g2, s2);
  };
  // The centred float64 sums of the rows of group g (held in s), published as round `round`
  // by the first thread of the second wavefront while the others go on (the first
  // wavefront gathers: the two halves of the exchange do not queue behind each other).
  // Every thread passes one barrier.
  constexpr int kPublisher = 64;
  auto sums_and_publish = [&](int64_t g, unsigned int round, Set& s) {
    TeamEntry* mine = &slot->entry[round & 3u][blockIdx.x];
    double* rd = red[round & 1u];
    double acc[K];
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const float kf = centre(s, r);
      const double kd = (double)kf;
      double s1 = 0.0, s2 = 0.0;
#pragma unroll
      for (int k = 0; k < V; ++k) {
        keep_packed(s.px[r * V + k]);
        // (a pack beyond the row or the tensor holds zeros, which are not x - k = 0)
        if (pk0 + k * BLOCK < npacks && g * R + r < M)
          add_centred_sums<T, E, RMS, true>(s.px[r * V + k], E, kf, kd, s1, s2);
      }
      acc[2 * r] = s1;
      acc[2 * r + 1] = s2;
    }
    // over the workgroup, in a fixed order; the publisher holds the result
#pragma unroll
    for (int k = 0; k < K; ++k) {
#pragma unroll
      for (int off = 32; off > 0; off >>= 1) acc[k] += __shfl_down(acc[k], off, 64);
    }
    const int wave = threadIdx.x >> 6;
    if ((threadIdx.x & 63) == 0) {
#pragma unroll
      for (int k = 0; k < K; ++k) rd[wave * K + k] = acc[k];
    }
    __syncthreads();
    if (threadIdx.x == kPublisher) {
#pragma unroll
      for (int k = 0; k < K; ++k) {
        double t = rd[k];
#pragma unroll
        for (int w = 1; w < BLOCK / 64; ++w) t += rd[w * K + k];
        acc[k] = t;
      }
      team_publish_f64<K>(mine, call_id, round, acc, lost != 0);
    }
  };
  // Y of group g (set s) from the statistics its round's gather left.  (g1 / s1, g2 / s2:
  // the groups of the other two sets, loaded again after the rare pass over whole rows so
  // that nothing stays live across that pass.)
  auto write = [&](int64_t g, unsigned int round, Set& s, int64_t g1, Set& s1, int64_t g2, Set& s2) {
    const int par = (int)(round & 1u);
    if (failed[par] != 0) {  // (uniform over the workgroup)
      // The team did not come together: the sums over the whole rows (X, which no
      // workgroup writes), then the packs again.
      for (int r = 0; r < R; ++r) {
        const T* xr = x + row_of(g, r) * (int64_t)N;
        const float kf = RMS ? 0.0f : split_row_centre(xr, (const T*)nullptr, N);
        double w1 = 0.0, w2 = 0.0;
        long_row_sums<T, E, BLOCK, RMS, false>(xr, (const T*)nullptr, N, 0, npacks, kf, w1, w2);
        __syncthreads();  // (red[] of the sum before has been read)
        block_sum2_f64<BLOCK>(w1, w2, red[0]);
        if (threadIdx.x == 0) set_stats(par, r, w1, w2, (double)kf);
      }
      __syncthreads();
      load_group(g, s);
      load_group(g1 >= 0 ? g1 : M, s1);  // (a group beyond the tensor: zeros)
      load_group(g2 >= 0 ? g2 : M, s2);
    }
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const int64_t row = g * R + r;
      const float hi = stat[par][r][0], lo = stat[par][r][1], rs = stat[par][r][2];
#pragma unroll
      for (int k = 0; k < V; ++k) {
        const bool held = pk0 + k * BLOCK < npacks;
        Pack<WT, E> gk;
        if constexpr (GL) {
          gk = gl[k][threadIdx.x];
        } else {
          keep_packed(pg[k]);  // (widened here, for this pack: not once ahead of the row loop)
          gk = pg[k];
        }
        if constexpr (!RMS) keep_packed(pb[k]);
        Pack<T, E> o;
#pragma unroll
        for (int i = 0; i < E; ++i) {
          float v;
          if constexpr (RMS)
            v = (s.px[r * V + k].get(i) * rs) * gk.get(i);
          else
            v = (((s.px[r * V + k].get(i) - hi) - lo) * rs) * gk.get(i) + pb[k].get(i);
          o.set(i, v);
        }
        if (held && row < M) o.store_stream(at(y + row * (int64_t)N + k * BLOCK * E, loff));
        // (the next pack is widened after this one has been stored, not before: registers)
        __builtin_amdgcn_sched_barrier(0);
      }
      if (c == 0 && threadIdx.x == 0 && row < M) {
        if constexpr (!RMS)
          if (mean) mean[row] = hi;
        if (rstd) rstd[row] = rs;
      }
    }
  };
  // One round: group g in set a (published a round ago) is gathered by the first wavefront
  // while the others request group g + 2 teams into set c and sum group g + teams in set
  // b; behind the barrier of that sum one thread publishes it and everyone writes Y of g.
  const bool first = threadIdx.x < 64;
  const int64_t st = teams;
  auto valid = [&](int64_t q) { return q < ngroups ? q : (int64_t)-1; };
  auto one_round = [&](int64_t g, unsigned int round, Set& a, Set& b, Set& cs) {
    const int64_t g1 = valid(g + st), g2 = valid(g + 2 * st);
    if (first)
      gather(g, round, a, g2, cs);
    else if (g2 >= 0)
      load_group(g2, cs);
    if (g1 >= 0)
      sums_and_publish(g1, round + 1, b);
    else
      __syncthreads();  // (the statistics of this round, for every thread)
    write(g, round, a, g1, b, g2, cs);
  };

  // Group j of the team (tm + j * teams) lives in register set j % 3: requested in round
  // j - 2, summed and published in round j - 1, gathered and written in round j.
  Set sa, sb, sc;
  int64_t g = tm;
  unsigned int round = 0;
  if (g < ngroups) {
    load_group(g, sa);
    if (g + st < ngroups) load_group(g + st, sb);
    sums_and_publish(g, 0, sa);
  }
  while (g < ngroups) {
    one_round(g, round, sa, sb, sc);
    g += st;
    ++round;
    if (g >= ngroups) break;
    one_round(g, round, sb, sc, sa);
    g += st;
    ++round;
    if (g >= ngroups) break;
    one_round(g, round, sc, sa, sb);
    g += st;
    ++round;
  }
}

// ---------------------------------------------------------------------------
// Split-row forward: few rows, each far beyond the registers (the regime of the
// reference's split-row kernels, Norm.h:632-812).  A row is cut into `chunks`
// chunks of `chunk_packs` packs (the last one takes the remainder as well, at
// most one workgroup stride more); workgroup (chunk, row) of the first launch
// sums its chunk, a second launch adds a row's partial sums in a fixed order and
// writes mean / rstd, a third normalizes chunk by chunk.
//
// Statistics.  The partial sums are sum(x - k) and sum((x - k)^2) accumulated in
// float64, k = the median of the row's first three elements (float32 and 16-bit
// values and their differences are exact in float64).  With 53-bit sums the
// subtraction s2 - s1*s1/N keeps 1e-10 of relative accuracy even when k lies a
// thousand standard deviations from the row (a padded head, outlier features),
// which single-precision shifted sums do not: rows of 3e5 elements around 100
// whose first three elements are 0 gave rstd 1e-4 off in float32.  It plays the
// part of the reference's Welford merge across work-groups (WelfordOps::combine,
// SharedReduceOps.h:71-88) with no division per element and no more passes over
// X.  The second launch forms mean = k + s1/N in float64 and splits it into
// hi = float(mean), which is the saved statistic, and lo = float(mean - hi); the
// third launch evaluates (x - hi) - lo, so the rounding of the saved mean never
// enters y, as in the resident kernel.  On a constant row x - k is exactly zero:
// mean is the constant and y is beta bit for bit.
//
// The partial sums and `lo` cross the launches in the first bytes of the chunk's
// own piece of Y (24 bytes, 8-byte aligned; every chunk is at least 1024 packs),
// which only that chunk's workgroup of the third launch overwrites, after it has
// read `lo`: no workspace, and no workgroup waits for another.
constexpr int kSplitSlotBytes = 24;

// `elems_per_chunk_pack`: elements of the row per pack (of the row type, whatever the
// element type of y).
template <class TY>
__device__ __forceinline__ double* split_chunk_slot(TY* y_row, int64_t first_pack,
                                                    int elems_per_chunk_pack) {
  return reinterpret_cast<double*>(
      (reinterpret_cast<uintptr_t>(y_row + first_pack * elems_per_chunk_pack) + 7) &
      ~uintptr_t(7));
}

// The packs [p0, p1) of chunk `chunk` out of `chunks`.
__device__ __forceinline__ void split_chunk_range(int chunk, int chunks, int64_t chunk_packs,
                                                  int64_t npacks, int64_t* p0, int64_t* p1) {
  *p0 = (int64_t)chunk * chunk_packs;
  *p1 = chunk == chunks - 1 ? npacks : *p0 + chunk_packs;
}

template <class T, int BLOCK, bool RMS, class TY = T>
__global__ void __launch_bounds__(BLOCK)
norm_fwd_split_sums_kernel(const T* __restrict__ x, const T* res, TY* __restrict__ y, int N,
                           int64_t chunk_packs) {
  constexpr int E = elems_per_pack<T>::value;
  __shared__ double red[2 * (BLOCK / 64)];
  const int64_t row = blockIdx.y;
  const T* xr = x + row * (int64_t)N;
  const T* rr = res ? res + row * (int64_t)N : nullptr;
  const int64_t npacks = ((int64_t)N + E - 1) / E;
  int64_t p0, p1;
  split_chunk_range(blockIdx.x, gridDim.x, chunk_packs, npacks, &p0, &p1);
  const float kf = RMS ? 0.0f : split_row_centre(xr, rr, N);
  double s1 = 0.0, s2 = 0.0;
  if (rr != nullptr)
    long_row_sums<T, E, BLOCK, RMS, true>(xr, rr, N, p0, p1, kf, s1, s2);
  else
    long_row_sums<T, E, BLOCK, RMS, false>(xr, rr, N, p0, p1, kf, s1, s2);
  block_sum2_f64<BLOCK>(s1, s2, red);
  if (threadIdx.x == 0) {
    double* slot = split_chunk_slot(y + row * (int64_t)N, p0, E);
    slot[0] = s1;
    slot[1] = s2;
  }
}

// One wavefront per row: lane l adds the partial sums of chunks l, l + 64, ...
// and a fixed tree adds the lanes, the same order on every run.
template <class T, bool RMS, class TY = T>
__global__ void __launch_bounds__(64)
norm_fwd_split_stats_kernel(const T* __restrict__ x, const T* res, TY* __restrict__ y,
                            float* __restrict__ mean, float* __restrict__ rstd, int N, int chunks,
                            int64_t chunk_packs, float eps) {
  constexpr int E = elems_per_pack<T>::value;
  const int64_t row = blockIdx.x;
  TY* yr = y + row * (int64_t)N;
  double s1 = 0.0, s2 = 0.0;
  for (int c = threadIdx.x; c < chunks; c += 64) {
    const double* slot = split_chunk_slot(yr, (int64_t)c * chunk_packs, E);
    s1 += slot[0];
    s2 += slot[1];
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    s1 += __shfl_down(s1, off, 64);
    s2 += __shfl_down(s2, off, 64);
  }
  s1 = __shfl(s1, 0, 64);
  s2 = __shfl(s2, 0, 64);
  const double dN = (double)N;
  float lo = 0.0f;
  if constexpr (RMS) {
    if (threadIdx.x == 0) rstd[row] = (float)(1.0 / sqrt(s2 / dN + (double)eps));
  } else {
    const double m1 = s1 / dN;
    const double mu = (double)split_row_centre(x + row * (int64_t)N,
                                               res ? res + row * (int64_t)N : nullptr, N) + m1;
    double var = (s2 - s1 * m1) / dN;
    var = var < 0.0 ? 0.0 : var;  // (a select: NaN stays NaN)
    const float hi = (float)mu;
    lo = (float)(mu - (double)hi);
    if (threadIdx.x == 0) {
      mean[row] = var == var ? hi : (float)var;  // NaN variance (a NaN or inf element): NaN mean
      rstd[row] = (float)(1.0 / sqrt(var + (double)eps));
    }
  }
  if constexpr (!RMS)
    for (int c = threadIdx.x; c < chunks; c += 64)
      *reinterpret_cast<float*>(split_chunk_slot(yr, (int64_t)c * chunk_packs, E)) = lo;
}

template <class T, class WT, int BLOCK, bool RMS, class TY = T>
__global__ void __launch_bounds__(BLOCK)
norm_fwd_split_apply_kernel(const T* __restrict__ x, const T* res, const WT* __restrict__ gamma,
                            const WT* __restrict__ beta, T* h, TY* __restrict__ y,
                            const float* __restrict__ mean, const float* __restrict__ rstd, int N,
                            int64_t chunk_packs) {
  constexpr int E = elems_per_pack<T>::value;
  const int64_t row = blockIdx.y;
  const T* xr = x + row * (int64_t)N;
  const T* rr = res ? res + row * (int64_t)N : nullptr;
  TY* yr = y + row * (int64_t)N;
  const int64_t npacks = ((int64_t)N + E - 1) / E;
  int64_t p0, p1;
  split_chunk_range(blockIdx.x, gridDim.x, chunk_packs, npacks, &p0, &p1);
  const float hi = RMS ? 0.0f : mean[row];
  const float rs = rstd[row];
  // the low part of the mean sits where this workgroup is about to write y
  const float lo = RMS ? 0.0f : *reinterpret_cast<const float*>(split_chunk_slot(yr, p0, E));
  __syncthreads();
  T* hr = rr != nullptr ? h + row * (int64_t)N : nullptr;
  if (rr != nullptr)
    long_row_apply<T, WT, TY, E, BLOCK, RMS, true>(xr, rr, gamma, beta, hr, yr, N, p0, p1, hi, lo,
                                                   rs);
  else
    long_row_apply<T, WT, TY, E, BLOCK, RMS, false>(xr, rr, gamma, beta, hr, yr, N, p0, p1, hi, lo,
                                                    rs);
}

// ---------------------------------------------------------------------------
// Backward, rows resident in registers: X and dY are read once, dX written
// once, and each lane keeps the dgamma/dbeta sums of its own columns in fp32
// registers over all the rows its workgroup visits.  At the end the BLOCK/G
// row slots of the workgroup are folded together through LDS in a fixed order
// and one fp32 row per workgroup goes to the [gridDim.x, N] partial buffers;
// colsum_finalize_kernel adds those up.
//
//   s1 = sum dy*gamma            s2 = sum dy*gamma*xhat       xhat = (x-mean)*rstd
//   dx = (rstd/N) * (N*gamma*dy - xhat*s2 - s1)               (RMS: mean = 0, no s1)
//   dgamma[j] = sum_rows dy*xhat   dbeta[j] = sum_rows dy
//
// ADD: dres, the gradient that reaches the normalized row by another path (the
// residual stream: the row was h = x + res and the loss also depends on h
// directly), is added to dx in float32 before the one rounding of the store.
// dres may be the memory of dx.
//
// PF (norm_bwd_prefetches()): the rows of the next iteration are requested
// before the arithmetic, the reduction and the stores of the current one, and
// wait in registers of their own.
template <class T, class WT, int G, int V, int BLOCK, int R, bool RMS, bool FAST,
          bool ADD = false>
__global__ void __launch_bounds__(BLOCK)
norm_bwd_resident_kernel(const T* __restrict__ dy, const T* __restrict__ x, const T* dres,
                         const float* __restrict__ mean, const float* __restrict__ rstd,
                         const WT* __restrict__ gamma, T* dx,
                         float* __restrict__ part_dg, float* __restrict__ part_db, int64_t M,
                         int N) {
  constexpr int E = elems_per_pack<T>::value;
  constexpr int RPB = BLOCK / G;  // row slots of the workgroup
  constexpr int RPI = RPB * R;    // rows per workgroup iteration (R per slot, see the forward)
  constexpr int FOLD_FLOATS = (RPB > 1) ? G * V * E : 1;
  __shared__ float red[reduce_lds_floats<G, BLOCK, 2 * R>::value];
  __shared__ float fold[FOLD_FLOATS];
  int phase = 0;
  const int slot = threadIdx.x / G;
  const int lane0 = threadIdx.x % G;
  const float fN = (float)N;
  const float inv_n = 1.0f / fN;
  const bool want_cols = part_dg != nullptr;  // uniform
  constexpr bool kWideWeights = V * E <= 16;  // few weights: widen to fp32 once, not per row
  constexpr bool PF = R == 1 && norm_bwd_prefetches((int)sizeof(T), G, V, FAST, RMS);
  // LDSG (norm_bwd_sums_in_lds()): rows of three or four packs a lane on 1024 lanes.
  // The registers hold the row, dY (twice: the next row is on its way) and the dbeta
  // sums; the dgamma sums live in LDS, each lane adding to its own 16-byte slots
  // (no other lane touches them, so no barrier), and gamma stays in memory, each
  // pack of it loaded (from L2) where it is used.
  constexpr bool LDSG = norm_bwd_sums_in_lds((int)sizeof(T), G, V, FAST);
  static_assert(!LDSG || (RPB == 1 && R == 1 && E == 8), "one 16-bit row a workgroup");
  __shared__ __attribute__((aligned(16))) float ldg[LDSG ? G * V * E : 4];
  // slot h (0, 1) of pack c of this lane: lanes side by side, 16 bytes each
  auto ldg_slot = [&](int c, int h) { return ldg + ((c * 2 + h) * G + lane0) * 4; };

  Pack<WT, E> gp[LDSG ? 1 : V];
  float dg[LDSG ? 1 : V][LDSG ? 1 : E];
  float db[RMS ? 1 : V][RMS ? 1 : E];
#pragma unroll
  for (int c = 0; c < V; ++c) {
    const int e0 = (c * G + lane0) * E;
    if constexpr (!LDSG)
      gp[c] = gamma ? load_row_pack<WT, E, false>(gamma, e0, N, true, 1.0f)
                    : Pack<WT, E>::splat(1.0f);
    if constexpr (LDSG) {
      *reinterpret_cast<float4*>(ldg_slot(c, 0)) = float4{0.0f, 0.0f, 0.0f, 0.0f};
      *reinterpret_cast<float4*>(ldg_slot(c, 1)) = float4{0.0f, 0.0f, 0.0f, 0.0f};
    }
#pragma unroll
    for (int i = 0; i < E; ++i) {
      if constexpr (!LDSG) dg[c][i] = 0.0f;
      if constexpr (!RMS) db[c][i] = 0.0f;
    }
  }
  // the weights of pack c, for the lane index `ln` (LDSG: made opaque per use, so the
  // pack offsets are not carried across the row loop)
  // (LDSG: a plain load, nothing conditional -- a test of the pointer is a branch around
  // the load, and the join of a branch waits for every request outstanding, the stores
  // of the packs before included.  Without gamma the load goes to the head of dY, which
  // such a row makes long enough, and its result is replaced.)
  const bool have_g = gamma != nullptr;
  const WT* wsrc = have_g ? gamma : reinterpret_cast<const WT*>(dy);
  auto weights = [&](int c, int ln) {
    if constexpr (LDSG) {
      Pack<WT, E> w =
          row_load<WT, E, false, true>(wsrc, have_g ? (c * G + ln) * E : 0, N, true, 1.0f);
      if (!have_g) w = Pack<WT, E>::splat(1.0f);
      return w;
    } else {
      return gp[c];
    }
  };

  const int64_t nrb = (M + RPI - 1) / RPI;
  // A row slot past the end of the tensor gets all-zero x and dy, so it adds
  // nothing to the column sums; its dx is not stored.
  bool ok[R];
  float mu[R], rs[R];
  Pack<T, E> xp[R][V], dp[R][V];
  auto fetch = [&](int64_t rb, bool (&fok)[R], float (&fmu)[R], float (&frs)[R],
                   Pack<T, E> (&fx)[R][V], Pack<T, E> (&fd)[R][V]) {
    const int64_t frow0 = (rb * RPB + slot) * R;
    const int lane = lane_again<LDSG || !FAST>(lane0);
    // (past the last row block the requests go to row 0 and are never used: a
    // branch around them measured 10-15 % slower over the whole kernel)
#pragma unroll
    for (int r = 0; r < R; ++r) {
      fok[r] = (RPI == 1 && !PF) ? true : (rb < nrb && frow0 + r < M);
      const int64_t rowc = fok[r] ? frow0 + r : 0;
      fmu[r] = RMS ? 0.0f : mean[rowc];
      frs[r] = rstd[rowc];
#pragma unroll
      for (int c = 0; c < V; ++c) {
        const int e0 = (c * G + lane) * E;
        fx[r][c] = row_load<T, E, true, FAST>(x + rowc * (int64_t)N, e0, N, fok[r], 0.0f);
        fd[r][c] = row_load<T, E, true, FAST>(dy + rowc * (int64_t)N, e0, N, fok[r], 0.0f);
      }
    }
  };
  if constexpr (PF) fetch(blockIdx.x, ok, mu, rs, xp, dp);
  for (int64_t rb = blockIdx.x; rb < nrb; rb += gridDim.x) {
    const int64_t row0 = (rb * RPB + slot) * R;
    // PF: the rows of the next iteration are requested before this iteration's
    // arithmetic, reduction and stores, and wait in registers of their own
    bool okn[PF ? R : 1];
    float mun[PF ? R : 1], rsn[PF ? R : 1];
    Pack<T, E> xn[PF ? R : 1][PF ? V : 1], dn[PF ? R : 1][PF ? V : 1];
    if constexpr (PF)
      fetch(rb + gridDim.x, okn, mun, rsn, xn, dn);
    else
      fetch(rb, ok, mu, rs, xp, dp);
    float acc[2 * R];
    // LDSG: the RMSNorm with three packs a lane has the registers to keep a row's
    // gamma packs from the row sums to dX (bf16 [8192, 18432] 190 -> 177 us, 24576:
    // 249 -> 221 us); with four packs, and in the LayerNorm, that spills and loses,
    // so they load them again
    constexpr bool kKeepG = LDSG && RMS && V == 3;
    Pack<WT, E> gk[kKeepG ? V : 1];
    const int lane = lane_again<LDSG || !FAST>(lane0);
#pragma unroll
    for (int r = 0; r < R; ++r) {
      // 16-bit rows: xhat = x*rs - mu*rs in one FMA (rounding far below a 16-bit
      // ulp); fp32 rows keep the cancellation-free (x - mu) * rs.
      const float nmr = -mu[r] * rs[r];
      acc[2 * r] = acc[2 * r + 1] = 0.0f;
#pragma unroll
      for (int c = 0; c < V; ++c) {
        if constexpr (!LDSG && !kWideWeights) keep_packed(gp[c]);
        const Pack<WT, E> gc = weights(c, lane);
        if constexpr (kKeepG) gk[c] = gc;
        float t[LDSG ? E : 1];
        if constexpr (LDSG) {
          if (want_cols) {
            const float4 t0 = *reinterpret_cast<const float4*>(ldg_slot(c, 0));
            const float4 t1 = *reinterpret_cast<const float4*>(ldg_slot(c, 1));
            t[0] = t0.x, t[1] = t0.y, t[2] = t0.z, t[3] = t0.w;
            t[4] = t1.x, t[5] = t1.y, t[6] = t1.z, t[7] = t1.w;
          }
        }
#pragma unroll
        for (int i = 0; i < E; ++i) {
          const float xv = xp[r][c].get(i);
          const float xh = RMS ? xv * rs[r]
                               : (sizeof(T) == 2 ? fmaf(xv, rs[r], nmr) : (xv - mu[r]) * rs[r]);
          const float gy = dp[r][c].get(i);
          const float g = gy * gc.get(i);
          if constexpr (!RMS) acc[2 * r] += g;
          acc[2 * r + 1] = fmaf(g, xh, acc[2 * r + 1]);
          if constexpr (LDSG)
            t[i] = fmaf(gy, xh, t[i]);
          else
            dg[c][i] = fmaf(gy, xh, dg[c][i]);
          if constexpr (!RMS) db[c][i] += gy;
        }
        if constexpr (LDSG) {
          if (want_cols) {
            *reinterpret_cast<float4*>(ldg_slot(c, 0)) = float4{t[0], t[1], t[2], t[3]};
            *reinterpret_cast<float4*>(ldg_slot(c, 1)) = float4{t[4], t[5], t[6], t[7]};
          }
        }
      }
    }
    group_allreduce<G, BLOCK, 2 * R, SumOp>(acc, red, phase);
    if (dx != nullptr) {
      const int ls = lane_after<LDSG || !FAST>(lane0, acc[1]);
#pragma unroll
      for (int r = 0; r < R; ++r) {
        T* dr = dx + (row0 + r) * (int64_t)N;
        // dx = (rs/N) * (N*g - xhat*s2 - s1), g = dy*gamma.  fp32 rows evaluate it
        // in this order (N*g - s1 cancels exactly where it should).  16-bit rows
        // use the regrouped rs*g - x*(rs*a) + (mu*rs*a - b), a = s2*rs/N,
        // b = s1*rs/N: two FMAs, rounding far below a 16-bit ulp.
        const float s1 = acc[2 * r], s2 = acc[2 * r + 1];
        const float term1 = row_mean_of<T>(rs[r], fN, inv_n);
        const float a = s2 * term1;
        const float b = RMS ? 0.0f : s1 * term1;
        const float ra = rs[r] * a;
        const float cc = mu[r] * ra - b;
        Pack<T, E> up[ADD ? V : 1];
        if constexpr (ADD) {
#pragma unroll
          for (int c = 0; c < V; ++c)
            up[c] = row_load<T, E, true, FAST>(dres + (ok[r] ? row0 + r : 0) * (int64_t)N,
                                               (c * G + ls) * E, N, ok[r], 0.0f);
        }
        // (LDSG, gamma looked up again: the weights of pack c + 1 are requested before
        // pack c is stored -- requests complete in order, so a lookup issued behind a
        // store would wait for that store)
        constexpr bool kAhead = LDSG && !kKeepG;
        Pack<WT, E> gahead;
        if constexpr (kAhead) gahead = weights(0, ls);
#pragma unroll
        for (int c = 0; c < V; ++c) {
          keep_packed(xp[r][c]);
          keep_packed(dp[r][c]);
          if constexpr (!LDSG && !kWideWeights) keep_packed(gp[c]);
          Pack<WT, E> gc;
          if constexpr (kAhead) {
            gc = gahead;
            if (c + 1 < V) gahead = weights(c + 1, ls);
            __builtin_amdgcn_sched_barrier(0);
          } else {
            gc = kKeepG ? gk[kKeepG ? c : 0] : weights(c, ls);
          }
          Pack<T, E> o;
#pragma unroll
          for (int i = 0; i < E; ++i) {
            const float g = dp[r][c].get(i) * gc.get(i);
            float f;
            if constexpr (sizeof(T) == 2) {
              f = fmaf(xp[r][c].get(i), -ra, fmaf(g, rs[r], cc));
            } else {
              const float xv = xp[r][c].get(i);
              const float xh = RMS ? xv * rs[r] : (xv - mu[r]) * rs[r];
              f = fN * g;
              f -= xh * s2;
              if constexpr (!RMS) f -= s1;
              f *= term1;
            }
            if constexpr (ADD) f += up[c].get(i);
            o.set(i, f);
          }
          row_store<T, E, true, FAST>(dr, (c * G + ls) * E, N, ok[r], o);
          if constexpr (kAhead) __builtin_amdgcn_sched_barrier(0);
        }
      }
    }
    if constexpr (PF) {
#pragma unroll
      for (int r = 0; r < R; ++r) {
        ok[r] = okn[r];
        mu[r] = mun[r];
        rs[r] = rsn[r];
#pragma unroll
        for (int c = 0; c < V; ++c) {
          xp[r][c] = xn[r][c];
          dp[r][c] = dn[r][c];
        }
      }
    }
  }

  if (!want_cols) return;
  // Fold the row slots that own the same columns, then emit one partial row.
  float* out_g = part_dg + (int64_t)blockIdx.x * N;
  float* out_b = RMS ? nullptr : part_db + (int64_t)blockIdx.x * N;
  if constexpr (RPB == 1) {
#pragma unroll
    for (int c = 0; c < V; ++c) {
      const int e0 = (c * G + lane0) * E;
      Pack<float, E> pg, pb;
      if constexpr (LDSG) {
        const float4 t0 = *reinterpret_cast<const float4*>(ldg_slot(c, 0));
        const float4 t1 = *reinterpret_cast<const float4*>(ldg_slot(c, 1));
        pg.set(0, t0.x), pg.set(1, t0.y), pg.set(2, t0.z), pg.set(3, t0.w);
        pg.set(4, t1.x), pg.set(5, t1.y), pg.set(6, t1.z), pg.set(7, t1.w);
      }
#pragma unroll
      for (int i = 0; i < E; ++i) {
        if constexpr (!LDSG) pg.set(i, dg[c][i]);
        if constexpr (!RMS) pb.set(i, db[c][i]);
      }
      store_row_pack<float, E, false>(out_g, e0, N, true, pg);
      if constexpr (!RMS) store_row_pack<float, E, false>(out_b, e0, N, true, pb);
    }
  } else {
    constexpr int NPASS = RMS ? 1 : 2;
#pragma unroll
    for (int pass = 0; pass < NPASS; ++pass) {
      // Row slots inside one wavefront (G < 64) are folded with shuffles first.
      if constexpr (G < 64) {
#pragma unroll
        for (int c = 0; c < V; ++c)
#pragma unroll
          for (int i = 0; i < E; ++i) {
            float v = pass == 0 ? dg[c][i] : db[RMS ? 0 : c][RMS ? 0 : i];
#pragma unroll
            for (int off = G; off < 64; off <<= 1) v += __shfl_xor(v, off, 64);
            if (pass == 0)
              dg[c][i] = v;
            else
              db[RMS ? 0 : c][RMS ? 0 : i] = v;
          }
      }
      constexpr int UNIT = G < 64 ? 64 : G;         // threads per fold unit
      constexpr int NUNIT = BLOCK / UNIT;           // units folded through LDS, in order
      const int unit = threadIdx.x / UNIT;
      const bool owner = (threadIdx.x % UNIT) < G;  // one lane group per unit holds the sums
#pragma unroll 1
      for (int u = 0; u < NUNIT; ++u) {
        if (unit == u && owner) {
#pragma unroll
          for (int c = 0; c < V; ++c) {
            const int e0 = (c * G + lane0) * E;
#pragma unroll
            for (int i = 0; i < E; ++i) {
              const float v = pass == 0 ? dg[c][i] : db[RMS ? 0 : c][RMS ? 0 : i];
              fold[e0 + i] = (u == 0) ? v : fold[e0 + i] + v;
            }
          }
        }
        __syncthreads();
      }
      float* out = pass == 0 ? out_g : out_b;
      for (int j = threadIdx.x; j < N; j += BLOCK) out[j] = fold[j];
      __syncthreads();
    }
  }
}

// ---------------------------------------------------------------------------
// The same backward for 16-bit rows that fill a layout exactly: N == G * V * E
// with G a whole number of wavefronts (not necessarily a power of two: hidden 5120
// is 320 lanes x 2 packs, 7168 is 448 x 2, 18432 is 768 x 3), every row slot of
// every row block holds a row (M % (BLOCK / G) == 0), and dx is written.
//
// No load and no store of the row loop is conditional.  In the kernel above a
// store sits behind a branch on the execution mask; the compiler cannot know
// whether it was issued, so its wait for the prefetched row -- older than that
// store, and the memory counter retires in order -- became a wait for the store as
// well: every iteration stalled until its predecessor's dX had reached L2.  Here a
// wait names exactly the operations that may stay in flight, and the rows of the
// next D - 1 iterations are on their way while the current one is worked on: the
// lane keeps D register sets and the row loop is unrolled D times, each copy of
// the body naming its sets statically (a register copy out of a set that is still
// being loaded would be a wait).  The row index is wavefront-uniform (a row slot
// is whole wavefronts), so row pointers are scalar arithmetic, mean / rstd are
// scalar loads and a lane adds a constant 32-bit offset.  One workgroup a compute
// unit (its lanes may take up to 256 registers): half the partial rows of the
// two-workgroup grid.  Arithmetic, summation order and partial rows are those of
// norm_bwd_resident_kernel, bit for bit for the same grid.
//
// Measured against norm_bwd_resident_kernel on one MI355X, bf16 rows x 16384
// (LayerNorm / RMSNorm, us): N = 2048 43.0 / 39.0 -> 40.5 / 37.6; 4096 74.5 / 69.9 ->
// 71.0 / 68.1; 5120 91.6 / 86.0 -> 89.3 / 85.3; 7168 125.6 / 120.4 -> 118.5 / 117.1;
// 8192 138.7 / 133.8 -> 134.5 / 130.6; LayerNorm 14336 250.9 -> 245.6 and 16384
// 285.4 -> 274.8 (with fp32 weights 266 -> 245 and 294 -> 275); 4096 rows of 4096:
// 28.1 / 25.2 -> 26.4 / 22.8.  Rows of 6144, 10240 and 12288 elements measured the
// same or slower than their three-pack layouts and keep those.
template <class T, class WT, int E, int V>
struct BwdRowSet {
  float mu, rs;
  Pack<T, E> x[V], d[V];
};

template <class T, class WT, int G, int V, int BLOCK, bool RMS, bool ADD, int D>
__global__ void __launch_bounds__(BLOCK)
norm_bwd_exact_kernel(const T* __restrict__ dy, const T* __restrict__ x, const T* dres,
                      const float* __restrict__ mean, const float* __restrict__ rstd,
                      const WT* __restrict__ gamma, T* dx, float* __restrict__ part_dg,
                      float* __restrict__ part_db, int64_t M, int N) {
  constexpr int E = elems_per_pack<T>::value;
  constexpr int RPB = BLOCK / G;  // row slots of the workgroup
  static_assert(G >= 64 && D >= 1 && sizeof(T) == 2, "16-bit rows on whole wavefronts");
  // the column sums of the row slots beyond the first, parked for the first to add
  constexpr int NSUMS = RMS ? 1 : 2;
  constexpr int FOLD_FLOATS = (RPB > 1) ? (RPB - 1) * NSUMS * G * V * E : 4;
  __shared__ float red[reduce_lds_floats<G, BLOCK, 2>::value];
  __shared__ __attribute__((aligned(16))) float fold[FOLD_FLOATS];
  int phase = 0;
  const int slot = threadIdx.x / G;
  const int lane0 = threadIdx.x % G;
  const float inv_n = 1.0f / (float)N;
  const bool want_cols = part_dg != nullptr;  // uniform
  constexpr bool kWideWeights = V * E <= 16;

  Pack<WT, E> gp[V];
  float dg[V][E];
  float db[RMS ? 1 : V][RMS ? 1 : E];
#pragma unroll
  for (int c = 0; c < V; ++c) {
    gp[c] = gamma ? Pack<WT, E>::load(gamma + (c * G + lane0) * E) : Pack<WT, E>::splat(1.0f);
#pragma unroll
    for (int i = 0; i < E; ++i) {
      dg[c][i] = 0.0f;
      if constexpr (!RMS) db[c][i] = 0.0f;
    }
  }

  const int64_t nrb = M / RPB;
  const int64_t step = gridDim.x;
  BwdRowSet<T, WT, E, V> ring[D];
  // (past the last row block the requests go to row block 0 and are never used)
  // A row slot is a whole number of wavefronts, so the row index is the same in
  // every lane of a wavefront: it lives in scalar registers, the row pointers are
  // scalar arithmetic, and a lane adds its constant 32-bit byte offset.
  const int slot_u = __builtin_amdgcn_readfirstlane(slot);
  uint32_t voff[V];
#pragma unroll
  for (int c = 0; c < V; ++c) voff[c] = (uint32_t)((c * G + lane0) * E * (int)sizeof(T));
  auto at = [](const T* rowp, uint32_t off) {
    return reinterpret_cast<const T*>(reinterpret_cast<const char*>(rowp) + off);
  };
  auto fetch = [&](int64_t rb, BwdRowSet<T, WT, E, V>& o) {
    const int64_t row = (rb < nrb ? rb : 0) * RPB + slot_u;
    o.mu = RMS ? 0.0f : mean[row];
    o.rs = rstd[row];
    const T* xr = x + row * (int64_t)N;
    const T* gr = dy + row * (int64_t)N;
#pragma unroll
    for (int c = 0; c < V; ++c) {
      o.x[c] = Pack<T, E>::load_stream(at(xr, voff[c]));
      o.d[c] = Pack<T, E>::load_stream(at(gr, voff[c]));
    }
  };
  auto work = [&](int64_t rb, BwdRowSet<T, WT, E, V>& w) {
    const int64_t row = rb * RPB + slot_u;
    const float mu = w.mu, rs = w.rs;
    const float nmr = -mu * rs;
    float acc[2] = {0.0f, 0.0f};
#pragma unroll
    for (int c = 0; c < V; ++c) {
      if constexpr (!kWideWeights) keep_packed(gp[c]);
#pragma unroll
      for (int i = 0; i < E; ++i) {
        const float xv = w.x[c].get(i);
        const float xh = RMS ? xv * rs : fmaf(xv, rs, nmr);
        const float gy = w.d[c].get(i);
        const float g = gy * gp[c].get(i);
        if constexpr (!RMS) acc[0] += g;
        acc[1] = fmaf(g, xh, acc[1]);
        dg[c][i] = fmaf(gy, xh, dg[c][i]);
        if constexpr (!RMS) db[c][i] += gy;
      }
    }
    group_allreduce<G, BLOCK, 2, SumOp>(acc, red, phase);
    T* dr = dx + row * (int64_t)N;
    const float s1 = acc[0], s2 = acc[1];
    const float term1 = rs * inv_n;
    const float a = s2 * term1;
    const float b = RMS ? 0.0f : s1 * term1;
    const float ra = rs * a;
    const float cc = mu * ra - b;
    Pack<T, E> up[ADD ? V : 1];
    if constexpr (ADD) {
#pragma unroll
      for (int c = 0; c < V; ++c)
        up[c] = Pack<T, E>::load_stream(at(dres + row * (int64_t)N, voff[c]));
    }
#pragma unroll
    for (int c = 0; c < V; ++c) {
      keep_packed(w.x[c]);
      keep_packed(w.d[c]);
      if constexpr (!kWideWeights) keep_packed(gp[c]);
      Pack<T, E> o;
#pragma unroll
      for (int i = 0; i < E; ++i) {
        const float g = w.d[c].get(i) * gp[c].get(i);
        float f = fmaf(w.x[c].get(i), -ra, fmaf(g, rs, cc));
        if constexpr (ADD) f += up[c].get(i);
        o.set(i, f);
      }
      o.store_stream(const_cast<T*>(at(dr, voff[c])));
    }
  };

#pragma unroll
  for (int k = 0; k < D - 1; ++k) fetch(blockIdx.x + k * step, ring[k]);
  int64_t rb = blockIdx.x;
  // whole groups of D row blocks as straight-line code: set k is worked on while the
  // set worked on before it is refilled with the row block D - 1 steps ahead
  while (rb + (D - 1) * step < nrb) {
#pragma unroll
    for (int k = 0; k < D; ++k) {
      fetch(rb + (D - 1) * step, ring[(k + D - 1) % D]);
      work(rb, ring[k]);
      rb += step;
    }
  }
  // at most D - 1 row blocks are left, and they have been requested
#pragma unroll
  for (int k = 0; k < D - 1; ++k) {
    if (rb < nrb) {  // uniform
      work(rb, ring[k]);
      rb += step;
    }
  }

  if (!want_cols) return;
  float* out_g = part_dg + (int64_t)blockIdx.x * N;
  float* out_b = RMS ? nullptr : part_db + (int64_t)blockIdx.x * N;
  if constexpr (RPB == 1) {
#pragma unroll
    for (int c = 0; c < V; ++c) {
      const int e0 = (c * G + lane0) * E;
      Pack<float, E> pg, pb;
#pragma unroll
      for (int i = 0; i < E; ++i) {
        pg.set(i, dg[c][i]);
        if constexpr (!RMS) pb.set(i, db[c][i]);
      }
      pg.store(out_g + e0);
      if constexpr (!RMS) pb.store(out_b + e0);
    }
  } else {
    // Row slots 1 .. RPB - 1 park their sums in LDS, 16 bytes a lane and half pack
    // (lanes side by side: no bank conflict), one barrier, and slot 0 adds them to its
    // own in slot order -- ((s0 + s1) + s2) + ..., the order of the kernel above -- and
    // writes the partial row with 128-bit stores.
    auto park = [&](int u, int which, int c, int h) {
      return reinterpret_cast<float4*>(fold) +
             ((((u - 1) * NSUMS + which) * V + c) * 2 + h) * G + lane0;
    };
    if (slot > 0) {
#pragma unroll
      for (int c = 0; c < V; ++c) {
        *park(slot, 0, c, 0) = float4{dg[c][0], dg[c][1], dg[c][2], dg[c][3]};
        *park(slot, 0, c, 1) = float4{dg[c][4], dg[c][5], dg[c][6], dg[c][7]};
        if constexpr (!RMS) {
          *park(slot, 1, c, 0) = float4{db[c][0], db[c][1], db[c][2], db[c][3]};
          *park(slot, 1, c, 1) = float4{db[c][4], db[c][5], db[c][6], db[c][7]};
        }
      }
    }
    __syncthreads();
    if (slot == 0) {
#pragma unroll
      for (int c = 0; c < V; ++c) {
        const int e0 = (c * G + lane0) * E;
        Pack<float, E> pg, pb;
#pragma unroll
        for (int i = 0; i < E; ++i) {
          pg.set(i, dg[c][i]);
          if constexpr (!RMS) pb.set(i, db[c][i]);
        }
#pragma unroll 1
        for (int u = 1; u < RPB; ++u) {
          const float4 g0 = *park(u, 0, c, 0), g1 = *park(u, 0, c, 1);
          pg.v[0] += g0.x, pg.v[1] += g0.y, pg.v[2] += g0.z, pg.v[3] += g0.w;
          pg.v[4] += g1.x, pg.v[5] += g1.y, pg.v[6] += g1.z, pg.v[7] += g1.w;
          if constexpr (!RMS) {
            const float4 b0 = *park(u, 1, c, 0), b1 = *park(u, 1, c, 1);
            pb.v[0] += b0.x, pb.v[1] += b0.y, pb.v[2] += b0.z, pb.v[3] += b0.w;
            pb.v[4] += b1.x, pb.v[5] += b1.y, pb.v[6] += b1.z, pb.v[7] += b1.w;
          }
        }
        pg.store(out_g + e0);
        if constexpr (!RMS) pb.store(out_b + e0);
      }
    }
  }
}

// What a lane of the long-row backward holds of one pack between request and use.
template <class T, class WT, int E>
struct LongRowBwdIn {
  Pack<T, E> x, dy, u;  // u: the gradient from the residual path (only with one)
  Pack<WT, E> g;
};

// acc[0] += sum dy*gamma, acc[1] += sum dy*gamma*xhat over the packs [p0, p1) of a thread.
template <class T, class WT, int E, int BLOCK, bool RMS>
__device__ __forceinline__ void long_row_bwd_sums(const T* xr, const T* gr, const WT* gamma, int N,
                                                  int64_t p0, int64_t p1, float mu, float rs,
                                                  float (&acc)[2]) {
  const bool hg = gamma != nullptr;  // uniform over the launch
  for_packs<kLongRowUnroll, BLOCK>(
      p0, p1, (int64_t)(N / E),
      [&](int64_t pk, auto whole) {
        constexpr bool W = decltype(whole)::value;
        LongRowBwdIn<T, WT, E> d;
        d.x = load_pack_of<T, E, false, W>(xr, pk * E, N, 0.0f);
        d.dy = load_pack_of<T, E, false, W>(gr, pk * E, N, 0.0f);
        d.g = hg ? load_pack_of<WT, E, false, W>(gamma, pk * E, N, 1.0f) : Pack<WT, E>::splat(1.0f);
        return d;
      },
      [&](int64_t, const LongRowBwdIn<T, WT, E>& d, auto) {
#pragma unroll
        for (int i = 0; i < E; ++i) {
          const float g = d.dy.get(i) * d.g.get(i);
          acc[0] += g;
          acc[1] = fmaf(g, (d.x.get(i) - mu) * rs, acc[1]);
        }
      });
}

// dx = (rs/N) * (N*gamma*dy - xhat*s2 - s1) (+ the residual path's gradient) over the
// packs [p0, p1) of a thread.
template <class T, class WT, int E, int BLOCK, bool RMS, bool HASRES>
__device__ __forceinline__ void long_row_bwd_dx(const T* xr, const T* gr, const T* ur,
                                                const WT* gamma, T* dr, int N, int64_t p0,
                                                int64_t p1, float mu, float rs, float s1,
                                                float s2) {
  const bool hg = gamma != nullptr;  // uniform over the launch
  const float fN = (float)N;
  const float term1 = rs / fN;
  for_packs<kLongRowUnroll, BLOCK>(
      p0, p1, (int64_t)(N / E),
      [&](int64_t pk, auto whole) {
        constexpr bool W = decltype(whole)::value;
        LongRowBwdIn<T, WT, E> d;
        d.x = load_pack_of<T, E, true, W>(xr, pk * E, N, 0.0f);
        d.dy = load_pack_of<T, E, true, W>(gr, pk * E, N, 0.0f);
        if constexpr (HASRES) d.u = load_pack_of<T, E, true, W>(ur, pk * E, N, 0.0f);
        d.g = hg ? load_pack_of<WT, E, false, W>(gamma, pk * E, N, 1.0f) : Pack<WT, E>::splat(1.0f);
        return d;
      },
      [&](int64_t pk, const LongRowBwdIn<T, WT, E>& d, auto whole) {
        constexpr bool W = decltype(whole)::value;
        Pack<T, E> o;
#pragma unroll
        for (int i = 0; i < E; ++i) {
          float f = fN * (d.dy.get(i) * d.g.get(i));
          f -= ((d.x.get(i) - mu) * rs) * s2;
          if constexpr (!RMS) f -= s1;
          f *= term1;
          if constexpr (HASRES) f += d.u.get(i);
          o.set(i, f);
        }
        store_pack_of<T, E, true, W>(dr, pk * E, N, o);
      });
}

// ---------------------------------------------------------------------------
// Backward dX for rows too wide for registers: one workgroup per row, two
// streaming passes over X and dY (sums, then dX).
template <class T, class WT, int BLOCK, bool RMS>
__global__ void __launch_bounds__(BLOCK)
norm_bwd_stream_dx_kernel(const T* __restrict__ dy, const T* __restrict__ x, const T* dres,
                          const float* __restrict__ mean, const float* __restrict__ rstd,
                          const WT* __restrict__ gamma, T* dx, int64_t M, int N) {
  constexpr int E = elems_per_pack<T>::value;
  __shared__ float red[reduce_lds_floats<BLOCK, BLOCK, 2>::value];
  int phase = 0;
  const int npacks = (N + E - 1) / E;
  for (int64_t row = blockIdx.x; row < M; row += gridDim.x) {
    const T* xr = x + row * (int64_t)N;
    const T* gr = dy + row * (int64_t)N;
    T* dr = dx + row * (int64_t)N;
    const float mu = RMS ? 0.0f : mean[row];
    const float rs = rstd[row];
    float acc[2] = {0.0f, 0.0f};
    long_row_bwd_sums<T, WT, E, BLOCK, RMS>(xr, gr, gamma, N, 0, npacks, mu, rs, acc);
    group_allreduce<BLOCK, BLOCK, 2, SumOp>(acc, red, phase);
    if (dres != nullptr)
      long_row_bwd_dx<T, WT, E, BLOCK, RMS, true>(xr, gr, dres + row * (int64_t)N, gamma, dr, N, 0,
                                                  npacks, mu, rs, acc[0], acc[1]);
    else
      long_row_bwd_dx<T, WT, E, BLOCK, RMS, false>(xr, gr, nullptr, gamma, dr, N, 0, npacks, mu, rs,
                                                   acc[0], acc[1]);
  }
}

// Split-row backward dX (see the split-row forward): workgroup (chunk, row) of
// the first launch leaves its chunk's s1 = sum dy*gamma and s2 = sum dy*gamma*xhat
// in split_ws[row][chunk]; every workgroup of the second launch adds its row's
// partial sums in the same fixed order and writes dX for its chunk.
template <class T, class WT, int BLOCK, bool RMS>
__global__ void __launch_bounds__(BLOCK)
norm_bwd_split_sums_kernel(const T* __restrict__ dy, const T* __restrict__ x,
                           const float* __restrict__ mean, const float* __restrict__ rstd,
                           const WT* __restrict__ gamma, float* __restrict__ split_ws, int N,
                           int64_t chunk_packs) {
  constexpr int E = elems_per_pack<T>::value;
  __shared__ float red[reduce_lds_floats<BLOCK, BLOCK, 2>::value];
  int phase = 0;
  const int64_t row = blockIdx.y;
  const T* xr = x + row * (int64_t)N;
  const T* gr = dy + row * (int64_t)N;
  const int64_t npacks = ((int64_t)N + E - 1) / E;
  int64_t p0, p1;
  split_chunk_range(blockIdx.x, gridDim.x, chunk_packs, npacks, &p0, &p1);
  const float mu = RMS ? 0.0f : mean[row];
  const float rs = rstd[row];
  float acc[2] = {0.0f, 0.0f};
  long_row_bwd_sums<T, WT, E, BLOCK, RMS>(xr, gr, gamma, N, p0, p1, mu, rs, acc);
  group_allreduce<BLOCK, BLOCK, 2, SumOp>(acc, red, phase);
  if (threadIdx.x == 0) {
    float* sc = split_ws + (row * gridDim.x + blockIdx.x) * 2;
    sc[0] = acc[0];
    sc[1] = acc[1];
  }
}

template <class T, class WT, int BLOCK, bool RMS>
__global__ void __launch_bounds__(BLOCK)
norm_bwd_split_dx_kernel(const T* __restrict__ dy, const T* __restrict__ x, const T* dres,
                         const float* __restrict__ mean, const float* __restrict__ rstd,
                         const WT* __restrict__ gamma, const float* __restrict__ split_ws,
                         T* dx, int N, int64_t chunk_packs) {
  constexpr int E = elems_per_pack<T>::value;
  static_assert(BLOCK >= kSplitMaxChunks, "one thread per partial sum");
  __shared__ float red[reduce_lds_floats<BLOCK, BLOCK, 2>::value];
  int phase = 0;
  const int64_t row = blockIdx.y;
  const T* xr = x + row * (int64_t)N;
  const T* gr = dy + row * (int64_t)N;
  T* dr = dx + row * (int64_t)N;
  const int64_t npacks = ((int64_t)N + E - 1) / E;
  int64_t p0, p1;
  split_chunk_range(blockIdx.x, gridDim.x, chunk_packs, npacks, &p0, &p1);
  const float mu = RMS ? 0.0f : mean[row];
  const float rs = rstd[row];
  float acc[2] = {0.0f, 0.0f};
  if (threadIdx.x < gridDim.x) {
    const float* sc = split_ws + (row * gridDim.x + threadIdx.x) * 2;
    acc[0] = sc[0];
    acc[1] = sc[1];
  }
  group_allreduce<BLOCK, BLOCK, 2, SumOp>(acc, red, phase);
  if (dres != nullptr)
    long_row_bwd_dx<T, WT, E, BLOCK, RMS, true>(xr, gr, dres + row * (int64_t)N, gamma, dr, N, p0,
                                                p1, mu, rs, acc[0], acc[1]);
  else
    long_row_bwd_dx<T, WT, E, BLOCK, RMS, false>(xr, gr, nullptr, gamma, dr, N, p0, p1, mu, rs,
                                                 acc[0], acc[1]);
}

// Split-row backward when dgamma / dbeta are wanted as well: one wavefront per
// row adds the row's chunk sums in a fixed order into totals[row] = {s1, s2} ...
template <int DUMMY = 0>
__global__ void __launch_bounds__(64)
norm_bwd_split_totals_kernel(const float* __restrict__ split_ws, float* __restrict__ totals,
                             int chunks) {
  const int64_t row = blockIdx.x;
  const float* sc = split_ws + row * (int64_t)chunks * 2;
  float s1 = 0.0f, s2 = 0.0f;
  for (int c = threadIdx.x; c < chunks; c += 64) {
    s1 += sc[2 * c];
    s2 += sc[2 * c + 1];
  }
  s1 = wave_group_allreduce<64, SumOp>(s1);
  s2 = wave_group_allreduce<64, SumOp>(s2);
  if (threadIdx.x == 0) {
    totals[2 * row] = s1;
    totals[2 * row + 1] = s2;
  }
}

// The column sums of one lane (E adjacent columns from e0) leave as whole packs: fp32 into
// a partial row, or, where the launch has one partial row only (`direct`), converted
// straight into dgamma / dbeta, which saves the second stage its launch and the fp32 row
// its trip through memory (bf16 [8, 4194304] LayerNorm backward: 86.7 us with the fp32 row
// written element by element and summed by a second stage).
template <class WT, int E>
__device__ __forceinline__ void store_column_sums(const float (&sum)[E], float* part_row, WT* out,
                                                  bool direct, int e0, int N) {
  if (direct) {
    if (out == nullptr) return;
    Pack<WT, E> o;
#pragma unroll
    for (int i = 0; i < E; ++i) o.set(i, sum[i]);
    store_row_pack<WT, E, false>(out, e0, N, true, o);
  } else {
#pragma unroll
    for (int h = 0; h < E; h += 4) {
      Pack<float, 4> o;
#pragma unroll
      for (int i = 0; i < 4; ++i) o.set(i, sum[h + i]);
      store_row_pack<float, 4, false>(part_row, e0 + h, N, true, o);
    }
  }
}

// ... and workgroup (bx, by) owns the BLOCK*E columns starting at bx*BLOCK*E and
// the rows by, by+gridDim.y, ...: it writes their dX and keeps the column sums
// of its strip, so X and dY are read once more, not twice (row `by` of the
// [gridDim.y, N] partial buffers, like the column-sum kernel below).  U rows are
// requested before any of them is used.
template <class T, class WT, int BLOCK, bool RMS>
__global__ void __launch_bounds__(BLOCK)
norm_bwd_split_dx_colsum_kernel(const T* __restrict__ dy, const T* __restrict__ x,
                                const T* dres, const float* __restrict__ mean,
                                const float* __restrict__ rstd, const WT* __restrict__ gamma,
                                const float* __restrict__ totals, T* dx,
                                float* __restrict__ part_dg, float* __restrict__ part_db,
                                WT* __restrict__ dgamma, WT* __restrict__ dbeta, int direct,
                                int64_t M, int N) {
  constexpr int E = elems_per_pack<T>::value;
  constexpr int U = 4;
  const int64_t e0l = ((int64_t)blockIdx.x * BLOCK + threadIdx.x) * E;
  if (e0l >= N) return;  // no barrier below
  const int e0 = (int)e0l;
  const Pack<WT, E> pg = gamma ? load_row_pack<WT, E, false>(gamma, e0, N, true, 1.0f)
                               : Pack<WT, E>::splat(1.0f);
  const float fN = (float)N;
  float dg[E], db[E];
#pragma unroll
  for (int i = 0; i < E; ++i) dg[i] = db[i] = 0.0f;
  for (int64_t row0 = blockIdx.y; row0 < M; row0 += (int64_t)gridDim.y * U) {
    Pack<T, E> px[U], pd[U], pu[U];
    float mu[U], rs[U], s1[U], s2[U];
    bool ok[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int64_t row = row0 + (int64_t)u * gridDim.y;
      ok[u] = row < M;
      const int64_t rc = ok[u] ? row : row0;
      px[u] = load_row_pack<T, E, true>(x + rc * (int64_t)N, e0, N, true, 0.0f);
      pd[u] = load_row_pack<T, E, true>(dy + rc * (int64_t)N, e0, N, true, 0.0f);
      pu[u] = Pack<T, E>::zero();
      if (dres != nullptr)
        pu[u] = load_row_pack<T, E, true>(dres + rc * (int64_t)N, e0, N, true, 0.0f);
      mu[u] = RMS ? 0.0f : mean[rc];
      rs[u] = rstd[rc];
      s1[u] = totals[2 * rc];
      s2[u] = totals[2 * rc + 1];
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      if (!ok[u]) continue;
      const int64_t row = row0 + (int64_t)u * gridDim.y;
      const float term1 = rs[u] / fN;
      Pack<T, E> o;
#pragma unroll
      for (int i = 0; i < E; ++i) {
        const float xh = (px[u].get(i) - mu[u]) * rs[u];
        float f = fN * (pd[u].get(i) * pg.get(i));
        f -= xh * s2[u];
        if constexpr (!RMS) f -= s1[u];
        o.set(i, f * term1 + pu[u].get(i));
        dg[i] = fmaf(pd[u].get(i), xh, dg[i]);
        db[i] += pd[u].get(i);
      }
      store_row_pack<T, E, true>(dx + row * (int64_t)N, e0, N, true, o);
    }
  }
  store_column_sums<WT, E>(dg, part_dg + (int64_t)blockIdx.y * N, dgamma, direct != 0, e0, N);
  if constexpr (!RMS)
    store_column_sums<WT, E>(db, part_db + (int64_t)blockIdx.y * N, dbeta, direct != 0, e0, N);
}

// Column sums for rows too wide for registers: workgroup (bx, by) owns the
// BLOCK*E columns starting at bx*BLOCK*E and the rows by, by+gridDim.y, ...;
// it writes row `by` of the [gridDim.y, N] partial buffers.
template <class T, class WT, int BLOCK, bool RMS>
__global__ void __launch_bounds__(BLOCK)
norm_bwd_stream_colsum_kernel(const T* __restrict__ dy, const T* __restrict__ x,
                              const float* __restrict__ mean, const float* __restrict__ rstd,
                              float* __restrict__ part_dg, float* __restrict__ part_db,
                              WT* __restrict__ dgamma, WT* __restrict__ dbeta, int direct,
                              int64_t M, int N) {
  constexpr int E = elems_per_pack<T>::value;
  const int e0 = (blockIdx.x * BLOCK + threadIdx.x) * E;
  if (e0 >= N) return;  // no barrier below
  float dg[E], db[E];
#pragma unroll
  for (int i = 0; i < E; ++i) dg[i] = db[i] = 0.0f;
  for (int64_t row = blockIdx.y; row < M; row += gridDim.y) {
    const float mu = RMS ? 0.0f : mean[row];
    const float rs = rstd[row];
    const Pack<T, E> px = load_row_pack<T, E, false>(x + row * (int64_t)N, e0, N, true, 0.0f);
    const Pack<T, E> pd = load_row_pack<T, E, false>(dy + row * (int64_t)N, e0, N, true, 0.0f);
#pragma unroll
    for (int i = 0; i < E; ++i) {
      dg[i] = fmaf(pd.get(i), (px.get(i) - mu) * rs, dg[i]);
      db[i] += pd.get(i);
    }
  }
  store_column_sums<WT, E>(dg, part_dg + (int64_t)blockIdx.y * N, dgamma, direct != 0, e0, N);
  if constexpr (!RMS)
    store_column_sums<WT, E>(db, part_db + (int64_t)blockIdx.y * N, dbeta, direct != 0, e0, N);
}

// ---------------------------------------------------------------------------
// Second stage of the dgamma/dbeta reduction: out[j] = sum_p part[p][j], rows
// added in a fixed order (deterministic).  A workgroup of 1024 threads covers
// 64 columns: 16 threads across, each owning 4 adjacent columns (one 16-byte
// load per partial row), 64 threads down striding over the P partial rows; the
// 64 row sums of a column are then added through LDS.  blockIdx.y selects
// dgamma (0) or dbeta (1).  Stands in for the at::sum(0) over the block
// buffers in the reference (LayerNormKernels.cpp:1312-1314).
constexpr int kFinalizeCols = 64;

//
// Very many partial rows under few columns (a GroupNorm over [N, C] with N in the hundreds of
// thousands: one partial row a sample, C / 64 workgroups) first FOLD: blockIdx.z takes the
// partial rows [z * fold_rows, (z + 1) * fold_rows) and leaves their fp32 sum in the first
// of them, in place (a workgroup reads and writes only its own columns of its own rows);
// the second launch then adds every fold_rows-th row (`row_stride` = fold_rows * N).
template <class WT, bool FOLD = false>
__global__ void __launch_bounds__(1024)
colsum_finalize_kernel(const float* part0, const float* part1, WT* __restrict__ out0,
                       WT* __restrict__ out1, int P, int N, int64_t row_stride = 0,
                       int fold_rows = 0) {
  constexpr int CQ = kFinalizeCols / 4, RL = 1024 / CQ;
  __shared__ float tile[RL][kFinalizeCols + 1];
  const float* part = blockIdx.y == 0 ? part0 : part1;
  WT* out = blockIdx.y == 0 ? out0 : out1;
  if (row_stride == 0) row_stride = N;
  if constexpr (FOLD) {
    if (part == nullptr) return;
    const int first = (int)blockIdx.z * fold_rows;
    part += (int64_t)first * row_stride;
    out = const_cast<WT*>(reinterpret_cast<const WT*>(part));  // (WT is float here)
    P = P - first < fold_rows ? P - first : fold_rows;
  }
  if (part == nullptr || out == nullptr) return;  // uniform per workgroup
  const int cq = threadIdx.x % CQ, rl = threadIdx.x / CQ;
  const int col0 = blockIdx.x * kFinalizeCols + cq * 4;
  // U partial rows per thread are requested before any of them is used, so the
  // 512 partial rows of a full-machine backward cost one memory round trip
  constexpr int U = 8;
  float a[4] = {0.0f, 0.0f, 0.0f, 0.0f};
  for (int p0 = rl; p0 < P; p0 += U * RL) {
    Pack<float, 4> v[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int p = p0 + u * RL;
      v[u] = load_row_pack<float, 4, false>(part + (int64_t)(p < P ? p : 0) * row_stride, col0, N,
                                            p < P, 0.0f);
    }
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
      for (int i = 0; i < 4; ++i) a[i] += v[u].get(i);
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) tile[rl][cq * 4 + i] = a[i];
  __syncthreads();
  if (threadIdx.x < kFinalizeCols) {
    const int col = blockIdx.x * kFinalizeCols + threadIdx.x;
    float s0 = 0.0f, s1 = 0.0f, s2 = 0.0f, s3 = 0.0f;
#pragma unroll
    for (int r = 0; r < RL; r += 4) {
      s0 += tile[r][threadIdx.x];
      s1 += tile[r + 1][threadIdx.x];
      s2 += tile[r + 2][threadIdx.x];
      s3 += tile[r + 3][threadIdx.x];
    }
    if (col < N) out[col] = (WT)((s0 + s1) + (s2 + s3));
  }
}

// The same sum for a handful of partial rows under very many columns (few, very
// long rows): a thread owns 4 adjacent columns and walks the P rows itself, so
// a workgroup of 256 threads covers 1024 columns and nothing crosses lanes.
constexpr int kFinalizeFlatRows = 16;
constexpr int kFinalizeFlatCols = 1024;

template <class WT>
__global__ void __launch_bounds__(256)
colsum_finalize_flat_kernel(const float* __restrict__ part0, const float* __restrict__ part1,
                            WT* __restrict__ out0, WT* __restrict__ out1, int P, int N) {
  const float* part = blockIdx.y == 0 ? part0 : part1;
  WT* out = blockIdx.y == 0 ? out0 : out1;
  if (part == nullptr || out == nullptr) return;  // uniform per workgroup
  const int col0 = (blockIdx.x * 256 + threadIdx.x) * 4;
  if (col0 >= N) return;
  float a[4] = {0.0f, 0.0f, 0.0f, 0.0f};
  for (int p = 0; p < P; ++p) {
    const Pack<float, 4> v = load_row_pack<float, 4, false>(part + (int64_t)p * N, col0, N, true,
                                                           0.0f);
#pragma unroll
    for (int i = 0; i < 4; ++i) a[i] += v.get(i);
  }
#pragma unroll
  for (int i = 0; i < 4; ++i)
    if (col0 + i < N) out[col0 + i] = (WT)a[i];
}

// ---------------------------------------------------------------------------
// Backward of rows beyond one workgroup's registers, dY and X read once: a team of workgroups
// holds R rows at a time, workgroup c of the team the packs [c * V * BLOCK, (c + 1) * V * BLOCK)
// of each -- V packs of dY and of X a lane and row, so a lane meets the same V * E columns in
// every row and its column sums (dgamma, dbeta) are 2 * V * E numbers however long the row is
// (kept in LDS).  The R rows' partial s1 = sum dy*gamma, s2 = sum dy*gamma*xhat cross the team
// in one exchange (team_publish_and_sum), every workgroup writes dX for what it holds, and the
// next R rows the team takes have been requested before the exchange began: two sets of R
// rows a lane, one being exchanged and written while the other arrives.  Team tm takes the
// row groups tm, tm + teams, ...; at the end each workgroup leaves its column sums in row
// tm of the [teams, N] partial buffers (the second stage adds them).  A workgroup whose wait
// runs out sums its R rows itself (dX must not overlap dY or X) and loads its packs again.
// One workgroup a compute unit: the two sets of rows take about 200 registers a lane.
template <class T, class WT, bool RMS, int R, int V>
__global__ void __launch_bounds__(kTeamBlock, kTeamBlock / 256)
norm_bwd_team_kernel(const T* __restrict__ dy, const T* __restrict__ x,
                     const float* __restrict__ mean, const float* __restrict__ rstd,
                     const WT* __restrict__ gamma, T* __restrict__ dx,
                     float* __restrict__ part_dg, float* __restrict__ part_db, int64_t M, int N,
                     int team, TeamSlot* slot, unsigned int call_id,
                     unsigned long long wait_ticks) {
  constexpr int E = elems_per_pack<T>::value;
  constexpr int BLOCK = kTeamBlock;
  constexpr int Q = E / 4;  // pieces of four floats in a pack's column sums
  __shared__ float red[reduce_lds_floats<BLOCK, BLOCK, 2 * R>::value];
  __shared__ float stat[2 * R + 1];  // the rows' s1, s2; whether the team failed
  // a lane's column sums, four floats a piece: piece q of pack k at colsum[(k * Q + q)][lane]
  // for dgamma, behind them the same for dbeta
  __shared__ Pack<float, 4> colsum[(RMS ? 1 : 2) * V * Q][BLOCK];
  int phase = 0;
  bool lost = false;  // (first wavefront) the workgroup has stopped waiting for its team
  const int tm = (int)blockIdx.x / team;
  const int c = (int)blockIdx.x - tm * team;
  const int teams = (int)gridDim.x / team;
  const int npacks = N / E;
  // pack k of the lane: pk0 + k * BLOCK of the row, held only if it lies in the row
  const int pk0 = c * (V * BLOCK) + (int)threadIdx.x;
  const int64_t ngroups = (M + R - 1) / R;
  const float fN = (float)N;
  Pack<WT, E> pg[V];
#pragma unroll
  for (int k = 0; k < V; ++k) {
    pg[k] = Pack<WT, E>::splat(1.0f);
    if (gamma != nullptr && pk0 + k * BLOCK < npacks)
      pg[k] = Pack<WT, E>::load(gamma + (int64_t)(pk0 + k * BLOCK) * E);
  }
#pragma unroll
  for (int q = 0; q < (RMS ? 1 : 2) * V * Q; ++q) colsum[q][threadIdx.x] = Pack<float, 4>::zero();

  // (a scalar pointer a row and one 32-bit byte offset a lane, formed as a pointer into
  // global memory: see norm_fwd_team_kernel)
  const uint32_t loff = (uint32_t)(pk0 < npacks ? pk0 : 0) * 16u;
  auto at = [](auto* p, uint32_t off) {
    using Elem = std::remove_pointer_t<decltype(p)>;
    typedef __attribute__((address_space(1))) Elem* GlobalPtr;
    return (Elem*)reinterpret_cast<GlobalPtr>(reinterpret_cast<uintptr_t>(p) + off);
  };
  // the lane's packs of the rows of group g (zeros beyond the tensor and beyond the row)
  auto load_group = [&](int64_t g, Pack<T, E> (&pd)[R * V], Pack<T, E> (&px)[R * V]) {
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const int64_t row = g * R + r;
#pragma unroll
      for (int k = 0; k < V; ++k) {
        pd[r * V + k] = Pack<T, E>::zero();
        px[r * V + k] = Pack<T, E>::zero();
        if (pk0 + k * BLOCK < npacks && row < M) {
          pd[r * V + k] = Pack<T, E>::load_stream(at(dy + row * (int64_t)N + k * BLOCK * E, loff));
          px[r * V + k] = Pack<T, E>::load_stream(at(x + row * (int64_t)N + k * BLOCK * E, loff));
        }
      }
    }
  };
  // The partial sums of the rows of group g (held in pd / px), published as round `round`.
  auto sums_and_publish = [&](int64_t g, unsigned int round, Pack<T, E> (&pd)[R * V],
                              Pack<T, E> (&px)[R * V]) {
    TeamEntry* mine = &slot->entry[round & 3u][blockIdx.x];
    float acc[2 * R];
#pragma unroll
    for (int r = 0; r < R; ++r) acc[2 * r] = acc[2 * r + 1] = 0.0f;
#pragma unroll
    for (int k = 0; k < V; ++k) {
#pragma unroll
      for (int r = 0; r < R; ++r) {
        const int64_t row = g * R + r < M ? g * R + r : M - 1;
        const float mu = RMS ? 0.0f : uniform_load<float>(mean + row);
        const float rs = uniform_load<float>(rstd + row);
#pragma unroll
        for (int i = 0; i < E; ++i) {
          const float gd = pd[r * V + k].get(i) * pg[k].get(i);
          acc[2 * r] += gd;
          acc[2 * r + 1] = fmaf(gd, (px[r * V + k].get(i) - mu) * rs, acc[2 * r + 1]);
        }
        keep_packed(pd[r * V + k]);
        keep_packed(px[r * V + k]);
        __builtin_amdgcn_sched_barrier(0);  // (one pack widened at a time: registers)
      }
    }
    group_allreduce<BLOCK, BLOCK, 2 * R, SumOp>(acc, red, phase);
    if (threadIdx.x == 0) team_publish_tagged<2 * R>(mine, call_id, round, acc, lost);
  };
  // The sums of group g (published as round `round`) across the team, its dX, its share of
  // the column sums; each pack's registers are given to the same pack of group gn (< 0:
  // none) as soon as its dX has been stored.  (go, po*: the group held in the other register
  // set, loaded again after the rare pass over whole rows so that nothing stays live
  // across that pass)
  auto finish = [&](int64_t g, unsigned int round, Pack<T, E> (&pd)[R * V], Pack<T, E> (&px)[R * V],
                    int64_t gn, int64_t go, Pack<T, E> (&pod)[R * V], Pack<T, E> (&pox)[R * V]) {
    // (every thread has read the stat[] of the round before: a team's last rounds have no
    // block reduction between two of these)
    __syncthreads();
    if (threadIdx.x < 64) {  // the first wavefront waits and adds up
      float tot[2 * R];
      const bool complete =
          team_gather_tagged<2 * R>(slot, slot->entry[round & 3u] + tm * team, team, call_id,
                                    round, wait_ticks, tot);
      lost = lost || !complete;
      if (threadIdx.x == 0) {
#pragma unroll
        for (int k = 0; k < 2 * R; ++k) stat[k] = tot[k];
        stat[2 * R] = complete ? 0.0f : 1.0f;
      }
    }
    __syncthreads();
    if (stat[2 * R] != 0.0f) {  // (uniform over the workgroup)
      // The team did not come together: the sums over the whole rows, then the packs again.
      // (one pack of each tensor a lane in flight: laid out for few registers, not for speed)
      for (int r = 0; r < R; ++r) {
        const int64_t row = g * R + r < M ? g * R + r : M - 1;
        const T* xr = x + row * (int64_t)N;
        const T* gr = dy + row * (int64_t)N;
        const float wmu = RMS ? 0.0f : mean[row], wrs = rstd[row];
        float ws[2] = {0.0f, 0.0f};
        for (int q = (int)threadIdx.x; q < npacks; q += BLOCK) {
          const Pack<T, E> qx = Pack<T, E>::load(xr + (int64_t)q * E);
          const Pack<T, E> qd = Pack<T, E>::load(gr + (int64_t)q * E);
          const Pack<WT, E> qg =
              gamma != nullptr ? Pack<WT, E>::load(gamma + (int64_t)q * E) : Pack<WT, E>::splat(1.0f);
#pragma unroll
          for (int i = 0; i < E; ++i) {
            const float gd = qd.get(i) * qg.get(i);
            ws[0] += gd;
            ws[1] = fmaf(gd, (qx.get(i) - wmu) * wrs, ws[1]);
          }
        }
        group_allreduce<BLOCK, BLOCK, 2, SumOp>(ws, red, phase);
        __syncthreads();  // (every thread has read stat[] before thread 0 rewrites it)
        if (threadIdx.x == 0) {
          stat[2 * r] = ws[0];
          stat[2 * r + 1] = ws[1];
        }
      }
      __syncthreads();
      load_group(g, pd, px);
      load_group(go >= 0 ? go : M, pod, pox);  // (a group beyond the tensor: zeros)
    }
#pragma unroll
    for (int k = 0; k < V; ++k) {
      const bool held = pk0 + k * BLOCK < npacks;
      // (the pack's column sums stay in registers over its R rows)
      Pack<float, 4> cg[Q], cb[Q];
#pragma unroll
      for (int q = 0; q < Q; ++q) {
        cg[q] = colsum[k * Q + q][threadIdx.x];
        if constexpr (!RMS) cb[q] = colsum[V * Q + k * Q + q][threadIdx.x];
      }
#pragma unroll
      for (int r = 0; r < R; ++r) {
        const int64_t row = g * R + r;
        const int64_t rowc = row < M ? row : M - 1;
        const float mu = RMS ? 0.0f : uniform_load<float>(mean + rowc);
        const float rs = uniform_load<float>(rstd + rowc);
        const float s1 = stat[2 * r], s2 = stat[2 * r + 1];
        const float term1 = rs / fN;
        Pack<T, E> o;
#pragma unroll
        for (int i = 0; i < E; ++i) {
          const float d = pd[r * V + k].get(i);
          const float xh = (px[r * V + k].get(i) - mu) * rs;
          float f = fN * (d * pg[k].get(i));
          f -= xh * s2;
          if constexpr (!RMS) f -= s1;
          o.set(i, f * term1);
          cg[i / 4].v[i % 4] = fmaf(d, xh, cg[i / 4].v[i % 4]);
          if constexpr (!RMS) cb[i / 4].v[i % 4] += d;
        }
        if (held && row < M)
          o.store_stream(at(dx + row * (int64_t)N + k * BLOCK * E, loff));
        // the registers go to the same pack of group gn
        if (gn >= 0) {
          const int64_t rown = gn * R + r;
          pd[r * V + k] = Pack<T, E>::zero();
          px[r * V + k] = Pack<T, E>::zero();
          if (held && rown < M) {
            pd[r * V + k] = Pack<T, E>::load_stream(at(dy + rown * (int64_t)N + k * BLOCK * E, loff));
            px[r * V + k] = Pack<T, E>::load_stream(at(x + rown * (int64_t)N + k * BLOCK * E, loff));
          }
        }
        // (the next pack is widened after this one has been stored, not before: registers)
        __builtin_amdgcn_sched_barrier(0);
      }
#pragma unroll
      for (int q = 0; q < Q; ++q) {
        colsum[k * Q + q][threadIdx.x] = cg[q];
        if constexpr (!RMS) colsum[V * Q + k * Q + q][threadIdx.x] = cb[q];
      }
    }
  };

  // Group j of the team (tm + j * teams) lives in register set j % 2: requested while group
  // j - 2 is written, summed and published one round before it is gathered and written, so
  // that neither the loads nor the exchange are waited for with nothing else to do.
  Pack<T, E> ad[R * V], ax[R * V], bd[R * V], bx[R * V];
  int64_t g = tm;
  unsigned int round = 0;
  if (g < ngroups) {
    load_group(g, ad, ax);
    if (g + teams < ngroups) load_group(g + teams, bd, bx);
    sums_and_publish(g, 0, ad, ax);
  }
  while (g < ngroups) {
    const int64_t g1 = g + teams, g2 = g + 2 * (int64_t)teams, g3 = g + 3 * (int64_t)teams;
    if (g1 < ngroups) sums_and_publish(g1, round + 1, bd, bx);
    finish(g, round, ad, ax, g2 < ngroups ? g2 : -1, g1 < ngroups ? g1 : -1, bd, bx);
    if (g1 >= ngroups) break;
    if (g2 < ngroups) sums_and_publish(g2, round + 2, ad, ax);
    finish(g1, round + 1, bd, bx, g3 < ngroups ? g3 : -1, g2 < ngroups ? g2 : -1, ad, ax);
    g = g2;
    round += 2;
  }
  if (part_dg != nullptr) {
#pragma unroll
    for (int k = 0; k < V; ++k) {
      if (pk0 + k * BLOCK >= npacks) continue;
      const int64_t e0 = (int64_t)(pk0 + k * BLOCK) * E;
      float* pgr = part_dg + (int64_t)tm * N + e0;
#pragma unroll
      for (int q = 0; q < Q; ++q) colsum[k * Q + q][threadIdx.x].store(pgr + 4 * q);
      if constexpr (!RMS) {
        float* pbr = part_db + (int64_t)tm * N + e0;
#pragma unroll
        for (int q = 0; q < Q; ++q) colsum[V * Q + k * Q + q][threadIdx.x].store(pbr + 4 * q);
      }
    }
  }
}

}  // namespace rownorm
