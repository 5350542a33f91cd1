// Last-dimension softmax / log_softmax forward and backward for gfx950, with
// the masked and "safe" variants.
//
// Same row layout as the norm kernels: G lanes share a row, each lane holds V
// 16-byte packs in registers, a workgroup handles BLOCK/G rows per iteration.
// Forward reads X once and writes Y once; backward reads Y and dY once and
// writes dX once.
//
// What they stand in for in the reference:
//   forward   DispatchSoftmaxForwardKernelFunctor (src/ATen/native/xpu/sycl/
//             SoftMaxKernels.cpp:212-410) and, for wide or misaligned rows,
//             SoftmaxForwardKernelFunctor (:546-684);
//   backward  DispatchSoftmaxBackwardKernelFunctor (:952-1102) and
//             SoftmaxBackwardKernelFunctor (:1229-1347).
// The arithmetic follows :300-357 (max, sum of exp(x - max), then
// exp(x-max)/sum or x - max - log(sum)) and :1031-1047 (y*(g - sum y*g) or
// g - exp(y)*sum g).
//
// Masked (is_masked in the reference, :257-272 and :991-1001): a boolean mask
// marks elements to leave out; forward treats them as -inf, backward treats the
// saved output there as 0.  The mask row that belongs to data row r is
// (r / div) * stride + r % mod, which covers a mask of the input's own shape
// (div 1, stride 1, mod 1), a [B, T] key-padding mask under [B, H, T, T] scores
// (div H*T, stride 1, mod 1), a [T, T] mask (stride 0, mod T) and a
// [B, 1, T, T] mask (div H*T, stride T, mod T).
// Safe (is_safe_softmax, :328-346): a row with no finite maximum comes out as
// zeros instead of NaN.
#pragma once
#include "device/pack.hpp"
#include "device/flat_rows.hpp"
#include "device/reduce.hpp"
#include "device/team.hpp"
#include "launch.hpp"
#include <type_traits>

namespace rownorm {

// exp for the accumulate type.  Rows stored in fp32 use the library expf (about
// one ulp); 16-bit rows tolerate the hardware exp2 path, whose relative error
// of a few times |x| * 2^-24 is far below half a 16-bit ulp.
template <bool PRECISE>
__device__ __forceinline__ float row_exp(float v) {
  if constexpr (PRECISE)
    return expf(v);
  else
    return __expf(v);
}

// Whether ragged rows of T are addressed through the 16-byte aligned window that
// holds them (window_head in device/pack.hpp).  16-bit rows: every ragged row
// starts 2-byte aligned, where a 128-bit access costs about twice an aligned
// one.  fp32 rows start 4-byte aligned, where it costs the same, and the
// window's second element-wise row end only slowed them (N = 4097: 4.9 -> 4.3
// TB/s), so they are addressed from the row start.
template <class T>
constexpr bool softmax_row_window() {
  return sizeof(T) == 2;
}

// A pack of a row of the multi-pass kernels: whole from the aligned window (to
// be trimmed), or through the general loader from the row start.
template <class T, int E, bool STREAM, bool WINDOW>
__device__ __forceinline__ Pack<T, E> stream_load(const T* row, int e0, int n, bool in_row,
                                                  float fill, int lo) {
  if constexpr (WINDOW)
    return load_window_pack<T, E, STREAM>(row, e0, n, in_row, fill);
  else
    return load_row_pack<T, E, STREAM>(row, e0, n, in_row, fill, lo);
}

// The kernels serve softmax and log_softmax (and the "safe" variant) from one
// instance, told apart by run-time flags that are uniform over the launch.  Each
// arm of such a choice opens with this marker: an empty volatile asm cannot be
// speculated, so the compiler keeps one scalar branch around the arm instead
// of computing both formulas for every element and selecting (which evaluated
// the exponential in log_softmax's output pass and in softmax's backward too).
#define ROWNORM_UNIFORM_ARM(tag) asm volatile("; " tag)

// Packs a thread of the multi-pass kernels requests before using the first.
constexpr int kStreamUnroll = 2;

// Rows of more than this many elements a lane are kept in storage format.
constexpr int kSoftmaxWideElems = 16;

struct MaskRef {
  const uint8_t* data;  // one byte per element, non-zero = masked out
  uint32_t div, mod;    // mask row of data row r: (r / div) * stride + r % mod
  int64_t stride;
};

// Start of the mask row for data row `r` (masked calls are limited to 2^31 rows).
__device__ __forceinline__ const uint8_t* mask_row_ptr(const MaskRef& m, int64_t r, int n) {
  const uint32_t r32 = (uint32_t)r;
  const int64_t mr = (int64_t)(r32 / m.div) * m.stride + (int64_t)(r32 % m.mod);
  return m.data + mr * (int64_t)n;
}

// E mask bytes for the pack starting at element e0 of a mask row whose elements are
// [lo, n) of `mrow` (fill: not masked).
template <int E, bool FAST>
__device__ __forceinline__ Pack<uint8_t, E> load_mask_pack(const uint8_t* mrow, int e0, int n,
                                                           bool ok, int lo = 0) {
  Pack<uint8_t, E> m;
  if constexpr (FAST) {
    const bool inb = e0 < n;
    m = Pack<uint8_t, E>::load(mrow + (inb ? e0 : 0));
    (void)ok;
  } else {
#pragma unroll
    for (int i = 0; i < E; ++i) m.v[i] = 0;
    if (ok) {
#pragma unroll
      for (int i = 0; i < E; ++i)
        if (e0 + i >= lo && e0 + i < n) m.v[i] = mrow[e0 + i];
    }
  }
  return m;
}

// Wavefronts per SIMD the register budget of the resident forward is set for (the
// second argument of __launch_bounds__ in HIP): eight, i.e. two 1024-thread
// workgroups a compute unit and 64 registers, for 1024-lane rows of 5..9 packs a
// lane; otherwise what the workgroup size implies.
constexpr int kSoftmaxFreshOffsetsMaxV = 9;
template <class TI, int G, int V, bool FAST, bool MASKED>
constexpr int softmax_fwd_min_blocks() {
  return (G == 1024 && FAST && !MASKED && V >= 5 && V <= kSoftmaxFreshOffsetsMaxV) ? 8 : 1;
}

template <class TI, class TO, int G, int V, int BLOCK, bool FAST, bool MASKED>
__global__ void __launch_bounds__(BLOCK, (softmax_fwd_min_blocks<TI, G, V, FAST, MASKED>()))
softmax_fwd_resident_kernel(const TI* __restrict__ x, TO* __restrict__ y, MaskRef mask, int64_t M,
                            int N, int flags) {
  constexpr int E = elems_per_pack<TI>::value;
  constexpr int RPB = BLOCK / G;
  constexpr bool PRECISE = sizeof(TO) == 4;
  constexpr bool WINDOW = !FAST && softmax_row_window<TI>();
  __shared__ float red[reduce_lds_floats<G, BLOCK, 1>::value];
  int phase = 0;
  const int slot = threadIdx.x / G;
  const int lane0 = threadIdx.x % G;
  const bool is_log = (flags & kSoftmaxLog) != 0;
  const bool is_safe = (flags & kSoftmaxSafe) != 0;
  const int64_t nrb = (M + RPB - 1) / RPB;
  for (int64_t rb = blockIdx.x; rb < nrb; rb += gridDim.x) {
    // The lane index is made opaque once a row and again before the stores: the
    // V pack offsets derive from it, and the compiler would otherwise compute
    // them all before the loop and hold a register or two a pack for the whole
    // kernel (at 8 and 9 packs a lane that decides whether two workgroups fit a
    // compute unit: 65536-element bf16 rows 220 -> 188 us, 73728 258 -> 215 us;
    // ragged rows drop from 94 to 54 registers).  From 10 packs a lane one
    // workgroup a compute unit is the better layout for log_softmax, and there
    // recomputing the offsets measured 1-2 % slower, so those keep them.
    constexpr bool kFreshOffsets =
        !(FAST && G == 1024 && V > kSoftmaxFreshOffsetsMaxV && V <= kMaxV);
    const int lane = lane_again<kFreshOffsets>(lane0);
    const int64_t row = rb * RPB + slot;
    const bool ok = RPB == 1 ? true : row < M;
    const int64_t rowc = ok ? row : 0;
    // ragged 16-bit rows go through the 16-byte aligned window that holds the row
    const int h = WINDOW ? window_head<TI, E>(x + rowc * (int64_t)N) : 0;
    const int nw = N + h;
    const TI* xr = x + rowc * (int64_t)N - h;
    TO* yr = y + row * (int64_t)N - h;
    Pack<TI, E> xp[V];
#pragma unroll
    for (int c = 0; c < V; ++c)
      xp[c] = row_load<TI, E, true, FAST>(xr, (c * G + lane) * E, nw, ok, -INFINITY, h, WINDOW);
#pragma unroll
    for (int c = 0; c < V; ++c)
      row_trim<TI, E, FAST>(xp[c], (c * G + lane) * E, nw, -INFINITY, h, WINDOW);
    if constexpr (V * E > kSoftmaxWideElems) {
      // Long rows (a vocabulary-sized row is 16 packs a lane): the row stays in
      // storage format and each of the three passes widens it again; softmax
      // then evaluates exp twice per element, log_softmax still once.
      if constexpr (MASKED) {
        const uint8_t* mrow = mask_row_ptr(mask, rowc, N) - h;
#pragma unroll
        for (int c = 0; c < V; ++c) {
          const Pack<uint8_t, E> mk =
              load_mask_pack<E, FAST>(mrow, (c * G + lane) * E, nw, ok, h);
#pragma unroll
          for (int i = 0; i < E; ++i)
            if (mk.v[i]) xp[c].set(i, -INFINITY);
        }
      }
      float mx[1] = {-INFINITY};
      float sum[1] = {0.0f};
      float m;
      if constexpr (!MASKED && FAST && V >= 8) {
        // the lane's packs in two halves, each with its own maximum and sum of
        // exp(x - maximum): the first half is worked on while the second is still
        // arriving, and the exponentials no longer wait for the block maximum
        constexpr int VA = V / 2;
        float m_t = -INFINITY, s_t = 0.0f;
        auto absorb = [&](auto c0, auto c1) {
          float pm = -INFINITY;
#pragma unroll
          for (int c = decltype(c0)::value; c < decltype(c1)::value; ++c)
#pragma unroll
            for (int i = 0; i < E; ++i) pm = fmaxf(pm, xp[c].get(i));
          const float nm = fmaxf(m_t, pm);
          // (nothing finite yet: the reference is 0, against which -inf elements add 0
          // and a NaN element still poisons the sum)
          const float ref = nm == -INFINITY ? 0.0f : nm;
          float acc = s_t * row_exp<PRECISE>(m_t - ref);
#pragma unroll
          for (int c = decltype(c0)::value; c < decltype(c1)::value; ++c) {
            keep_packed(xp[c]);
#pragma unroll
            for (int i = 0; i < E; ++i) acc += row_exp<PRECISE>(xp[c].get(i) - ref);
          }
          s_t = acc;
          m_t = nm;
        };
        absorb(std::integral_constant<int, 0>{}, std::integral_constant<int, VA>{});
        absorb(std::integral_constant<int, VA>{}, std::integral_constant<int, V>{});
        mx[0] = m_t;
        group_allreduce<G, BLOCK, 1, MaxOp>(mx, red, phase);
        m = mx[0];
        // exp(-inf - m) = 0 drops lanes that saw nothing finite; a row with no finite
        // element at all gives NaN, like the three-pass form
        sum[0] = s_t == 0.0f ? (m == -INFINITY ? NAN : 0.0f) : s_t * row_exp<PRECISE>(m_t - m);
        group_allreduce<G, BLOCK, 1, SumOp>(sum, red, phase);
      } else {
#pragma unroll
        for (int c = 0; c < V; ++c)
#pragma unroll
          for (int i = 0; i < E; ++i) mx[0] = fmaxf(mx[0], xp[c].get(i));
        group_allreduce<G, BLOCK, 1, MaxOp>(mx, red, phase);
        m = mx[0];
#pragma unroll
        for (int c = 0; c < V; ++c) {
          keep_packed(xp[c]);
#pragma unroll
          for (int i = 0; i < E; ++i) sum[0] += row_exp<PRECISE>(xp[c].get(i) - m);
        }
        group_allreduce<G, BLOCK, 1, SumOp>(sum, red, phase);
      }
      if (is_log) {
        ROWNORM_UNIFORM_ARM("log_softmax: x - max - log(sum)");
        float k = logf(sum[0]);
        const int ls = lane_after<kFreshOffsets>(lane0, k);
#pragma unroll
        for (int c = 0; c < V; ++c) {
          keep_packed(xp[c]);
          Pack<TO, E> o;
#pragma unroll
          for (int i = 0; i < E; ++i) o.set(i, (xp[c].get(i) - m) - k);
          row_store<TO, E, true, FAST>(yr, (c * G + ls) * E, nw, ok, o, h);
        }
      } else if (is_safe) {
        ROWNORM_UNIFORM_ARM("safe softmax: zeros for a row without a finite element");
        float k = 1.0f / sum[0];
        const int ls = lane_after<kFreshOffsets>(lane0, k);
        const bool zero_row = m == -INFINITY;
#pragma unroll
        for (int c = 0; c < V; ++c) {
          keep_packed(xp[c]);
          Pack<TO, E> o;
#pragma unroll
          for (int i = 0; i < E; ++i)
            o.set(i, zero_row ? 0.0f : row_exp<PRECISE>(xp[c].get(i) - m) * k);
          row_store<TO, E, true, FAST>(yr, (c * G + ls) * E, nw, ok, o, h);
        }
      } else {
        ROWNORM_UNIFORM_ARM("softmax: exp(x - max) / sum");
        float k = 1.0f / sum[0];
        const int ls = lane_after<kFreshOffsets>(lane0, k);
#pragma unroll
        for (int c = 0; c < V; ++c) {
          keep_packed(xp[c]);
          Pack<TO, E> o;
#pragma unroll
          for (int i = 0; i < E; ++i) o.set(i, row_exp<PRECISE>(xp[c].get(i) - m) * k);
          row_store<TO, E, true, FAST>(yr, (c * G + ls) * E, nw, ok, o, h);
        }
      }
      continue;
    }
    float xf[V][E];
#pragma unroll
    for (int c = 0; c < V; ++c)
#pragma unroll
      for (int i = 0; i < E; ++i) xf[c][i] = xp[c].get(i);
    if constexpr (MASKED) {
      const uint8_t* mrow = mask_row_ptr(mask, rowc, N) - h;
#pragma unroll
      for (int c = 0; c < V; ++c) {
        const Pack<uint8_t, E> mk = load_mask_pack<E, FAST>(mrow, (c * G + lane) * E, nw, ok, h);
#pragma unroll
        for (int i = 0; i < E; ++i) xf[c][i] = mk.v[i] ? -INFINITY : xf[c][i];
      }
    }
    float mx[1] = {-INFINITY};
#pragma unroll
    for (int c = 0; c < V; ++c)
#pragma unroll
      for (int i = 0; i < E; ++i) mx[0] = fmaxf(mx[0], xf[c][i]);
    group_allreduce<G, BLOCK, 1, MaxOp>(mx, red, phase);
    const float m = mx[0];
    float sum[1] = {0.0f};
    // (no arm markers here: both arms evaluate exp(x - max) and differ in what
    // they keep, which the compiler turns into one shared body by itself)
    if (is_log) {
      // keep x - max; the exponentials only feed the sum
#pragma unroll
      for (int c = 0; c < V; ++c)
#pragma unroll
        for (int i = 0; i < E; ++i) {
          xf[c][i] -= m;
          sum[0] += row_exp<PRECISE>(xf[c][i]);
        }
    } else {
#pragma unroll
      for (int c = 0; c < V; ++c)
#pragma unroll
        for (int i = 0; i < E; ++i) {
          xf[c][i] = row_exp<PRECISE>(xf[c][i] - m);
          sum[0] += xf[c][i];
        }
    }
    group_allreduce<G, BLOCK, 1, SumOp>(sum, red, phase);
    if (is_log) {
      ROWNORM_UNIFORM_ARM("log_softmax: (x - max) - log(sum)");
      float k = logf(sum[0]);
      const int ls = lane_after<kFreshOffsets>(lane0, k);
#pragma unroll
      for (int c = 0; c < V; ++c) {
        Pack<TO, E> o;
#pragma unroll
        for (int i = 0; i < E; ++i) o.set(i, xf[c][i] - k);
        row_store<TO, E, true, FAST>(yr, (c * G + ls) * E, nw, ok, o, h);
      }
    } else if (is_safe) {
      ROWNORM_UNIFORM_ARM("safe softmax: zeros for a row without a finite element");
      float k = 1.0f / sum[0];
      const int ls = lane_after<kFreshOffsets>(lane0, k);
      const bool zero_row = m == -INFINITY;
#pragma unroll
      for (int c = 0; c < V; ++c) {
        Pack<TO, E> o;
#pragma unroll
        for (int i = 0; i < E; ++i) o.set(i, zero_row ? 0.0f : xf[c][i] * k);
        row_store<TO, E, true, FAST>(yr, (c * G + ls) * E, nw, ok, o, h);
      }
    } else {
      ROWNORM_UNIFORM_ARM("softmax: exp(x - max) * (1 / sum)");
      float k = 1.0f / sum[0];
      const int ls = lane_after<kFreshOffsets>(lane0, k);
#pragma unroll
      for (int c = 0; c < V; ++c) {
        Pack<TO, E> o;
#pragma unroll
        for (int i = 0; i < E; ++i) o.set(i, xf[c][i] * k);
        row_store<TO, E, true, FAST>(yr, (c * G + ls) * E, nw, ok, o, h);
      }
    }
  }
}

// Rows too wide for registers: one workgroup per row, two passes over the row.
// The first keeps a running maximum and a running sum of exp(x - maximum) per
// thread, rescaling the sum whenever a pack raises the maximum; the threads'
// pairs are merged with s * exp(m - M) after the block maximum M is known.  The
// second pass writes the output.  (The reference's SoftmaxForwardKernelFunctor,
// SoftMaxKernels.cpp:546-684, walks the row three times: max, sum, output.)
template <class TI, class TO, int BLOCK, bool MASKED>
__global__ void __launch_bounds__(BLOCK)
softmax_fwd_stream_kernel(const TI* __restrict__ x, TO* __restrict__ y, MaskRef mask, int64_t M,
                          int N, int flags) {
  constexpr int E = elems_per_pack<TI>::value;
  constexpr bool PRECISE = sizeof(TO) == 4;
  constexpr bool WINDOW = softmax_row_window<TI>();
  __shared__ float red[reduce_lds_floats<BLOCK, BLOCK, 1>::value];
  int phase = 0;
  const bool is_log = (flags & kSoftmaxLog) != 0;
  const bool is_safe = (flags & kSoftmaxSafe) != 0;
  for (int64_t row = blockIdx.x; row < M; row += gridDim.x) {
    // 16-bit rows: the 16-byte aligned window that holds the row, elements [h, nw) of it
    const int h = WINDOW ? window_head<TI, E>(x + row * (int64_t)N) : 0;
    const int nw = N + h;
    const int npacks = (nw + E - 1) / E;
    const TI* xr = x + row * (int64_t)N - h;
    TO* yr = y + row * (int64_t)N - h;
    const uint8_t* mrow = MASKED ? mask_row_ptr(mask, row, N) - h : nullptr;
    // element i of a pack, with the mask applied
    auto masked_value = [&](const Pack<TI, E>& p, const Pack<uint8_t, E>& mk, int i) {
      const float v = p.get(i);
      if constexpr (MASKED) return mk.v[i] ? -INFINITY : v;
      return v;
    };
    float m_t = -INFINITY, s_t = 0.0f;
    // kStreamUnroll packs a thread are requested before the first is used
    for (int pk0 = threadIdx.x; pk0 < npacks; pk0 += kStreamUnroll * BLOCK) {
      Pack<TI, E> pv[kStreamUnroll];
      Pack<uint8_t, E> mv[kStreamUnroll];
#pragma unroll
      for (int u = 0; u < kStreamUnroll; ++u) {
        const int pk = pk0 + u * BLOCK;
        pv[u] = stream_load<TI, E, false, WINDOW>(xr, pk * E, nw, pk < npacks, -INFINITY, h);
        if constexpr (MASKED) mv[u] = load_mask_pack<E, false>(mrow, pk * E, nw, pk < npacks, h);
      }
#pragma unroll
      for (int u = 0; u < kStreamUnroll; ++u) {
        if constexpr (WINDOW) trim_window_pack<TI, E>(pv[u], (pk0 + u * BLOCK) * E, nw, -INFINITY, h);
        float v[E];
        float pm = -INFINITY;
#pragma unroll
        for (int i = 0; i < E; ++i) {
          v[i] = masked_value(pv[u], mv[u], i);
          pm = fmaxf(pm, v[i]);
        }
        // bring the sum so far to the new maximum and add the pack -- without a branch
        // (a lane-divergent branch here costs registers and keeps loads from overlapping):
        // while nothing finite has been seen the reference is 0, against which -inf
        // elements add 0 and a NaN element still poisons the row
        const float nm = fmaxf(m_t, pm);
        const float ref = nm == -INFINITY ? 0.0f : nm;
        float acc = s_t * row_exp<PRECISE>(m_t - ref);
#pragma unroll
        for (int i = 0; i < E; ++i) acc += row_exp<PRECISE>(v[i] - ref);
        s_t = acc;
        m_t = nm;
      }
    }
    float mx[1] = {m_t};
    group_allreduce<BLOCK, BLOCK, 1, MaxOp>(mx, red, phase);
    const float m = mx[0];
    // exp(-inf - m) = 0 drops threads that saw nothing finite; a row with no
    // finite element at all gives exp(NaN) = NaN, like the three-pass form
    float sum[1] = {s_t == 0.0f ? (m == -INFINITY ? NAN : 0.0f) : s_t * row_exp<PRECISE>(m_t - m)};
    group_allreduce<BLOCK, BLOCK, 1, SumOp>(sum, red, phase);
    const float k = is_log ? logf(sum[0]) : 1.0f / sum[0];
    const bool zero_row = is_safe && m == -INFINITY;
    for (int pk0 = threadIdx.x; pk0 < npacks; pk0 += kStreamUnroll * BLOCK) {
      Pack<TI, E> pv[kStreamUnroll];
      Pack<uint8_t, E> mv[kStreamUnroll];
#pragma unroll
      for (int u = 0; u < kStreamUnroll; ++u) {
        const int pk = pk0 + u * BLOCK;
        pv[u] = stream_load<TI, E, true, WINDOW>(xr, pk * E, nw, pk < npacks, -INFINITY, h);
        if constexpr (MASKED) mv[u] = load_mask_pack<E, false>(mrow, pk * E, nw, pk < npacks, h);
      }
#pragma unroll
      for (int u = 0; u < kStreamUnroll; ++u) {
        const int pk = pk0 + u * BLOCK;
        Pack<TO, E> o;
        if (is_log) {
          ROWNORM_UNIFORM_ARM("log_softmax");
#pragma unroll
          for (int i = 0; i < E; ++i) o.set(i, (masked_value(pv[u], mv[u], i) - m) - k);
        } else {
          ROWNORM_UNIFORM_ARM("softmax");
#pragma unroll
          for (int i = 0; i < E; ++i) {
            const float v = row_exp<PRECISE>(masked_value(pv[u], mv[u], i) - m) * k;
            o.set(i, zero_row ? 0.0f : v);
          }
        }
        store_row_pack<TO, E, true>(yr, pk * E, nw, pk < npacks, o, h);
      }
    }
  }
}

// ---------------------------------------------------------------------------
// Forward for few, very long rows of whole packs (fewer rows than half the compute units;
// 16-byte aligned X and Y, no mask): a row is held in the registers of a team of
// workgroups, as in the norm forward for rows beyond the registers (norm_fwd_team_kernel).
// The grid is at most two workgroups of 512 threads a compute unit, all resident at once;
// workgroup b belongs to team b / team and keeps chunk b % team of the team's current
// row, V packs a lane.  It finds its chunk's maximum m_c and s_c = sum exp(x - m_c),
// publishes the pair and waits (bounded) for its team's pairs (device/team.hpp); each
// workgroup then merges them in chunk order -- M = max m_c, S = sum s_c * exp(m_c - M),
// the same values in every workgroup, run to run -- and writes its chunk of the output
// out of its registers.  X is read once, and the whole machine works on a handful of
// rows, where one workgroup a row (the reference's layout for such rows,
// SoftMaxKernels.cpp:546-684, and softmax_fwd_stream_kernel here) leaves most compute
// units idle.  A workgroup whose wait runs out takes the whole row's maximum and sum
// itself (a second pass over X, which no workgroup writes: Y must not overlap X), loads
// its chunk again and goes on; every wave reaches the end of the kernel whatever the
// other workgroups do.
template <class TI, class TO, int V>
__global__ void __launch_bounds__(kTeamBlock, kTeamPerCu * kTeamBlock / 256)
softmax_fwd_team_kernel(const TI* __restrict__ x, TO* __restrict__ y, int64_t M, int N, int flags,
                        int team, int64_t chunk_packs, TeamSlot* slot, unsigned int call_id,
                        unsigned long long wait_ticks) {
  constexpr int E = elems_per_pack<TI>::value;
  constexpr int BLOCK = kTeamBlock;
  constexpr bool PRECISE = sizeof(TO) == 4;
  __shared__ float red[reduce_lds_floats<BLOCK, BLOCK, 1>::value];
  __shared__ double tpart[kTeamMaxWorkgroups][2];
  __shared__ float stat[4];  // the row's maximum, 1 / sum or log(sum), -, whether the team failed
  int phase = 0;
  const bool is_log = (flags & kSoftmaxLog) != 0;
  const bool is_safe = (flags & kSoftmaxSafe) != 0;
  const int tm = (int)blockIdx.x / team;
  const int c = (int)blockIdx.x - tm * team;
  const int teams = (int)gridDim.x / team;
  const int npacks = N / E;
  const int64_t p0 = (int64_t)c * chunk_packs;
  const int64_t p1 = p0 + chunk_packs < npacks ? p0 + chunk_packs : npacks;
  const int nloc = p1 > p0 ? (int)(p1 - p0) : 0;  // packs of this chunk
  const bool full = nloc == V * BLOCK;  // (uniform) all chunks but a row's last
  const int64_t pbase = nloc > 0 ? p0 : 0;
  const uint32_t loff = (uint32_t)(threadIdx.x * 16);
  const uint32_t ooff = (uint32_t)(threadIdx.x * E * sizeof(TO));
  // (the sum is formed as a pointer into global memory: a pointer made from an integer
  // is otherwise a generic one, and generic accesses wait for everything outstanding)
  auto at = [](auto* p, uint32_t off) {
    using Elem = std::remove_pointer_t<decltype(p)>;
    typedef __attribute__((address_space(1))) Elem* GlobalPtr;
    return (Elem*)reinterpret_cast<GlobalPtr>(reinterpret_cast<uintptr_t>(p) + off);
  };
  unsigned int round = 0;
  for (int64_t row = tm; row < M; row += teams, ++round) {
    TeamEntry* entries = slot->entry[round & 1u];
    if (threadIdx.x == 0) team_store(&entries[blockIdx.x].tag, 0ull);
    const TI* xr = x + row * (int64_t)N;
    const TI* xb = xr + pbase * E;
    Pack<TI, E> xp[V];
    auto load_chunk = [&]() {
      if (full) {
        // (straight-line code: V requests in flight a lane, nothing conditional)
#pragma unroll
        for (int k = 0; k < V; ++k) xp[k] = Pack<TI, E>::load_stream(at(xb + k * BLOCK * E, loff));
      } else {
#pragma unroll
        for (int k = 0; k < V; ++k) {
          xp[k] = Pack<TI, E>::splat(-INFINITY);
          if (k * BLOCK + (int)threadIdx.x < nloc)
            xp[k] = Pack<TI, E>::load_stream(at(xb + k * BLOCK * E, loff));
        }
      }
    };
    load_chunk();
    float pm = -INFINITY;
#pragma unroll
    for (int k = 0; k < V; ++k)
#pragma unroll
      for (int i = 0; i < E; ++i) pm = fmaxf(pm, xp[k].get(i));
    // (the chunk stays in storage format across the reductions and the wait)
#pragma unroll
    for (int k = 0; k < V; ++k) keep_packed(xp[k]);
    float mx[1] = {pm};
    group_allreduce<BLOCK, BLOCK, 1, MaxOp>(mx, red, phase);
    const float m_c = mx[0];
    // (nothing finite in the chunk: against 0, -inf elements add 0 and NaN still poisons)
    const float ref = m_c == -INFINITY ? 0.0f : m_c;
    float acc = 0.0f;
#pragma unroll
    for (int k = 0; k < V; ++k)
#pragma unroll
      for (int i = 0; i < E; ++i) acc += row_exp<PRECISE>(xp[k].get(i) - ref);
#pragma unroll
    for (int k = 0; k < V; ++k) keep_packed(xp[k]);
    float sm[1] = {acc};
    group_allreduce<BLOCK, BLOCK, 1, SumOp>(sm, red, phase);
    if (threadIdx.x < 64) {  // the first wavefront publishes, waits and merges
      const int lane = (int)threadIdx.x;
      const bool complete = team_publish_and_gather(slot, entries, tm, team, call_id, round,
                                                    wait_ticks, (double)m_c, (double)sm[0], tpart);
      // (the lanes of a wavefront see one another's LDS stores in program order)
      if (complete) {
        float mm = -INFINITY;
        for (int j = lane; j < team; j += 64) mm = fmaxf(mm, (float)tpart[j][0]);
        mm = wave_group_allreduce<64, MaxOp>(mm);
        // a chunk with nothing finite adds 0; a row with nothing finite gives NaN, as
        // exp(-inf - -inf) does in the three-pass form
        float ss = 0.0f;
        for (int j = lane; j < team; j += 64) {
          const float mj = (float)tpart[j][0], sj = (float)tpart[j][1];
          ss += sj == 0.0f ? (mm == -INFINITY ? NAN : 0.0f) : sj * row_exp<PRECISE>(mj - mm);
        }
        ss = wave_group_allreduce<64, SumOp>(ss);
        if (lane == 0) {
          stat[0] = mm;
          stat[1] = is_log ? logf(ss) : 1.0f / ss;
          stat[3] = 0.0f;
        }
      } else if (lane == 0) {
        stat[3] = 1.0f;
      }
    }
    __syncthreads();
    if (stat[3] != 0.0f) {  // (uniform over the workgroup)
      // The team did not come together: the running maximum and sum of the whole row, as
      // softmax_fwd_stream_kernel takes them, then the chunk again, whose registers the pass
      // over the row has used.
      float m_t = -INFINITY, s_t = 0.0f;
      for (int pk0 = threadIdx.x; pk0 < npacks; pk0 += kStreamUnroll * BLOCK) {
        Pack<TI, E> pv[kStreamUnroll];
#pragma unroll
        for (int u = 0; u < kStreamUnroll; ++u) {
          const int pk = pk0 + u * BLOCK;
          pv[u] = Pack<TI, E>::splat(-INFINITY);
          if (pk < npacks) pv[u] = Pack<TI, E>::load(xr + (int64_t)pk * E);
        }
#pragma unroll
        for (int u = 0; u < kStreamUnroll; ++u) {
          float q = -INFINITY;
#pragma unroll
          for (int i = 0; i < E; ++i) q = fmaxf(q, pv[u].get(i));
          const float nm = fmaxf(m_t, q);
          const float rf = nm == -INFINITY ? 0.0f : nm;
          float a2 = s_t * row_exp<PRECISE>(m_t - rf);
#pragma unroll
          for (int i = 0; i < E; ++i) a2 += row_exp<PRECISE>(pv[u].get(i) - rf);
          s_t = a2;
          m_t = nm;
        }
      }
      float wm[1] = {m_t};
      group_allreduce<BLOCK, BLOCK, 1, MaxOp>(wm, red, phase);
      float ws[1] = {s_t == 0.0f ? (wm[0] == -INFINITY ? NAN : 0.0f)
                                 : s_t * row_exp<PRECISE>(m_t - wm[0])};
      group_allreduce<BLOCK, BLOCK, 1, SumOp>(ws, red, phase);
      if (threadIdx.x == 0) {
        stat[0] = wm[0];
        stat[1] = is_log ? logf(ws[0]) : 1.0f / ws[0];
      }
      __syncthreads();
      load_chunk();
    }
    const float m = stat[0], kk = stat[1];
    const bool zero_row = is_safe && m == -INFINITY;
    TO* yb = y + row * (int64_t)N + pbase * E;
#pragma unroll
    for (int k = 0; k < V; ++k) {
      if (full || k * BLOCK + (int)threadIdx.x < nloc) {
        Pack<TO, E> o;
        if (is_log) {
          ROWNORM_UNIFORM_ARM("log_softmax");
#pragma unroll
          for (int i = 0; i < E; ++i) o.set(i, (xp[k].get(i) - m) - kk);
        } else {
          ROWNORM_UNIFORM_ARM("softmax");
#pragma unroll
          for (int i = 0; i < E; ++i) {
            const float v = row_exp<PRECISE>(xp[k].get(i) - m) * kk;
            o.set(i, zero_row ? 0.0f : v);
          }
        }
        o.store_stream(at(yb + k * BLOCK * E, ooff));
      }
    }
    // stat[] is rewritten for the next row only after every thread has passed the
    // barriers of the next block reductions, i.e. after it has read this row's values
  }
}

// Backward.  TG: dtype of grad and of y (the saved forward output); TO: dtype
// of the input gradient.
template <class TG, class TO, int G, int V, int BLOCK, bool FAST, bool MASKED>
__global__ void __launch_bounds__(BLOCK)
softmax_bwd_resident_kernel(const TG* __restrict__ grad, const TG* __restrict__ y,
                            TO* __restrict__ gi, MaskRef mask, int64_t M, int N, int flags) {
  constexpr int E = elems_per_pack<TG>::value;
  constexpr int RPB = BLOCK / G;
  constexpr bool PRECISE = sizeof(TO) == 4 && sizeof(TG) == 4;
  constexpr bool WINDOW = !FAST && softmax_row_window<TG>();
  __shared__ float red[reduce_lds_floats<G, BLOCK, 1>::value];
  int phase = 0;
  const int slot = threadIdx.x / G;
  const int lane0 = threadIdx.x % G;
  const bool is_log = (flags & kSoftmaxLog) != 0;
  // y's packs are aligned like grad's when the two base addresses are congruent
  const bool y_whole = WINDOW && same_pack_alignment(grad, y);
  // 16-bit rows of more than 4 packs a lane on 1024 lanes: both tensors stay in storage
  // format across the reduction and are widened again for the output (as fp32 copies
  // they would take 16 registers a pack)
  constexpr bool kPacked = FAST && !MASKED && G == 1024 && V > 4 && sizeof(TG) == 2;
  const int64_t nrb = (M + RPB - 1) / RPB;
  for (int64_t rb = blockIdx.x; rb < nrb; rb += gridDim.x) {
    // ragged rows: opaque once a row and again before the stores (see the forward;
    // 8192 x 4097 bf16 49.6 -> 41.8 us); whole-pack rows measured 1 % slower with it
    const int lane = lane_again<!FAST || kPacked>(lane0);
    const int64_t row = rb * RPB + slot;
    const bool ok = RPB == 1 ? true : row < M;
    const int64_t rowc = ok ? row : 0;
    // ragged 16-bit rows go through the 16-byte aligned window that holds the row of grad
    const int h = WINDOW ? window_head<TG, E>(grad + rowc * (int64_t)N) : 0;
    const int nw = N + h;
    const TG* gr = grad + rowc * (int64_t)N - h;
    const TG* yr = y + rowc * (int64_t)N - h;
    TO* outr = gi + row * (int64_t)N - h;
    Pack<TG, E> pg[V], py[V];
#pragma unroll
    for (int c = 0; c < V; ++c) {
      const int e0 = (c * G + lane) * E;
      pg[c] = row_load<TG, E, true, FAST>(gr, e0, nw, ok, 0.0f, h, WINDOW);
      py[c] = row_load<TG, E, true, FAST>(yr, e0, nw, ok, 0.0f, h, y_whole);
    }
#pragma unroll
    for (int c = 0; c < V; ++c) {
      const int e0 = (c * G + lane) * E;
      row_trim<TG, E, FAST, true>(pg[c], e0, nw, 0.0f, h, WINDOW);
      row_trim<TG, E, FAST, true>(py[c], e0, nw, 0.0f, h, y_whole);
    }
    if constexpr (kPacked) {
      float sum[1] = {0.0f};
      if (is_log) {
        ROWNORM_UNIFORM_ARM("log_softmax backward: sum of grad");
#pragma unroll
        for (int c = 0; c < V; ++c)
#pragma unroll
          for (int i = 0; i < E; ++i) sum[0] += pg[c].get(i);
      } else {
        ROWNORM_UNIFORM_ARM("softmax backward: sum of y * grad");
#pragma unroll
        for (int c = 0; c < V; ++c)
#pragma unroll
          for (int i = 0; i < E; ++i) sum[0] = fmaf(py[c].get(i), pg[c].get(i), sum[0]);
      }
      group_allreduce<G, BLOCK, 1, SumOp>(sum, red, phase);
      float s = sum[0];
      const int ls = lane_after<true>(lane0, s);
#pragma unroll
      for (int c = 0; c < V; ++c) {
        keep_packed(pg[c]);
        keep_packed(py[c]);
        Pack<TO, E> o;
#pragma unroll
        for (int i = 0; i < E; ++i) {
          const float gv = pg[c].get(i), yv = py[c].get(i);
          o.set(i, is_log ? gv - row_exp<PRECISE>(yv) * s : yv * (gv - s));
        }
        row_store<TO, E, true, FAST>(outr, (c * G + ls) * E, nw, ok, o, h);
      }
      continue;
    }
    float gf[V][E], yf[V][E];
#pragma unroll
    for (int c = 0; c < V; ++c)
#pragma unroll
      for (int i = 0; i < E; ++i) {
        gf[c][i] = pg[c].get(i);
        yf[c][i] = py[c].get(i);
      }
    if constexpr (MASKED) {
      const uint8_t* mrow = mask_row_ptr(mask, rowc, N) - h;
#pragma unroll
      for (int c = 0; c < V; ++c) {
        const Pack<uint8_t, E> mk = load_mask_pack<E, FAST>(mrow, (c * G + lane) * E, nw, ok, h);
#pragma unroll
        for (int i = 0; i < E; ++i) yf[c][i] = mk.v[i] ? 0.0f : yf[c][i];
      }
    }
    float sum[1] = {0.0f};
    if (is_log) {
      ROWNORM_UNIFORM_ARM("log_softmax backward: sum of grad");
#pragma unroll
      for (int c = 0; c < V; ++c)
#pragma unroll
        for (int i = 0; i < E; ++i) sum[0] += gf[c][i];
    } else {
      ROWNORM_UNIFORM_ARM("softmax backward: sum of y * grad");
#pragma unroll
      for (int c = 0; c < V; ++c)
#pragma unroll
        for (int i = 0; i < E; ++i) sum[0] = fmaf(yf[c][i], gf[c][i], sum[0]);
    }
    group_allreduce<G, BLOCK, 1, SumOp>(sum, red, phase);
    float s = sum[0];
    const int ls = lane_after<!FAST>(lane0, s);
    if (is_log) {
      ROWNORM_UNIFORM_ARM("log_softmax backward: grad - exp(y) * sum");
#pragma unroll
      for (int c = 0; c < V; ++c) {
        Pack<TO, E> o;
#pragma unroll
        for (int i = 0; i < E; ++i) o.set(i, gf[c][i] - row_exp<PRECISE>(yf[c][i]) * s);
        row_store<TO, E, true, FAST>(outr, (c * G + ls) * E, nw, ok, o, h);
      }
    } else {
      ROWNORM_UNIFORM_ARM("softmax backward: y * (grad - sum)");
#pragma unroll
      for (int c = 0; c < V; ++c) {
        Pack<TO, E> o;
#pragma unroll
        for (int i = 0; i < E; ++i) o.set(i, yf[c][i] * (gf[c][i] - s));
        row_store<TO, E, true, FAST>(outr, (c * G + ls) * E, nw, ok, o, h);
      }
    }
  }
}

// ---------------------------------------------------------------------------
// Short ragged rows through LDS: see device/flat_rows.hpp.
template <class T, int G, int VP, int BLOCK, int LDSB>
__global__ void __launch_bounds__(BLOCK)
softmax_fwd_flat_kernel(const T* __restrict__ x, T* __restrict__ y, int64_t M, int N,
                        int chunk_rows, int flags) {
  constexpr int E = elems_per_pack<T>::value;
  constexpr int RPB = BLOCK / G;
  constexpr bool PRECISE = sizeof(T) == 4;
  constexpr int U = LDSB / (BLOCK * 16);
  __shared__ __attribute__((aligned(16))) T buf[LDSB / sizeof(T) + E];
  const bool is_log = (flags & kSoftmaxLog) != 0;
  const bool is_safe = (flags & kSoftmaxSafe) != 0;
  const int64_t row0 = (int64_t)blockIdx.x * chunk_rows;
  const int rows_here = M - row0 < chunk_rows ? (int)(M - row0) : chunk_rows;
  const int nelem = rows_here * N;
  flat_stage_in<T, BLOCK, U>(x + row0 * (int64_t)N, buf, nelem);
  __syncthreads();
  const int lane = threadIdx.x % G;
  for (int r = threadIdx.x / G; r < rows_here; r += RPB) {
    T* rowb = buf + r * N;
    float v[VP][E];
    float m = -INFINITY;
#pragma unroll
    for (int c = 0; c < VP; ++c) {
      const int j = (c * G + lane) * E;
      Pack<T, E> p = Pack<T, E>::splat(-INFINITY);
      if (j < N) p = flat_row_pack<T, E>(rowb, j);
#pragma unroll
      for (int i = 0; i < E; ++i) {
        v[c][i] = j + i < N ? p.get(i) : -INFINITY;
        m = fmaxf(m, v[c][i]);
      }
    }
    m = wave_group_allreduce<G, MaxOp>(m);
    float sum = 0.0f;
    if (is_log) {
      ROWNORM_UNIFORM_ARM("log_softmax: (x - max) - log(sum)");
#pragma unroll
      for (int c = 0; c < VP; ++c)
#pragma unroll
        for (int i = 0; i < E; ++i) {
          v[c][i] -= m;
          sum += row_exp<PRECISE>(v[c][i]);
        }
    } else {
#pragma unroll
      for (int c = 0; c < VP; ++c)
#pragma unroll
        for (int i = 0; i < E; ++i) {
          v[c][i] = row_exp<PRECISE>(v[c][i] - m);
          sum += v[c][i];
        }
    }
    sum = wave_group_allreduce<G, SumOp>(sum);
    const float kf = is_log ? logf(sum) : 1.0f / sum;
    const bool zero_row = is_safe && m == -INFINITY;
#pragma unroll
    for (int c = 0; c < VP; ++c) {
      const int j = (c * G + lane) * E;
      Pack<T, E> o;
#pragma unroll
      for (int i = 0; i < E; ++i)
        o.set(i, is_log ? v[c][i] - kf : (zero_row ? 0.0f : v[c][i] * kf));
      if (j < N) flat_row_store<T, E>(rowb, j, N - j, o);
    }
  }
  __syncthreads();
  flat_stage_out<T, BLOCK, U>(y + row0 * (int64_t)N, buf, nelem);
}

template <class T, int G, int VP, int BLOCK, int LDSB>
__global__ void __launch_bounds__(BLOCK)
softmax_bwd_flat_kernel(const T* __restrict__ grad, const T* __restrict__ y, T* __restrict__ gi,
                        int64_t M, int N, int chunk_rows, int flags) {
  constexpr int E = elems_per_pack<T>::value;
  constexpr int RPB = BLOCK / G;
  constexpr bool PRECISE = sizeof(T) == 4;
  constexpr int U = LDSB / (BLOCK * 16);
  __shared__ __attribute__((aligned(16))) T bg[LDSB / sizeof(T) + E];
  __shared__ __attribute__((aligned(16))) T by[LDSB / sizeof(T) + E];
  const bool is_log = (flags & kSoftmaxLog) != 0;
  const int64_t row0 = (int64_t)blockIdx.x * chunk_rows;
  const int rows_here = M - row0 < chunk_rows ? (int)(M - row0) : chunk_rows;
  const int nelem = rows_here * N;
  flat_stage_in2<T, BLOCK, U>(grad + row0 * (int64_t)N, bg, y + row0 * (int64_t)N, by, nelem);
  __syncthreads();
  const int lane = threadIdx.x % G;
  for (int r = threadIdx.x / G; r < rows_here; r += RPB) {
    T* rg = bg + r * N;
    const T* ry = by + r * N;
    float gf[VP][E], yf[VP][E];
    float sum = 0.0f;
#pragma unroll
    for (int c = 0; c < VP; ++c) {
      const int j = (c * G + lane) * E;
      Pack<T, E> pg = Pack<T, E>::zero(), py = Pack<T, E>::zero();
      if (j < N) {
        pg = flat_row_pack<T, E>(rg, j);
        py = flat_row_pack<T, E>(ry, j);
      }
#pragma unroll
      for (int i = 0; i < E; ++i) {
        gf[c][i] = j + i < N ? pg.get(i) : 0.0f;
        yf[c][i] = j + i < N ? py.get(i) : 0.0f;
        sum = is_log ? sum + gf[c][i] : fmaf(yf[c][i], gf[c][i], sum);
      }
    }
    sum = wave_group_allreduce<G, SumOp>(sum);
#pragma unroll
    for (int c = 0; c < VP; ++c) {
      const int j = (c * G + lane) * E;
      Pack<T, E> o;
#pragma unroll
      for (int i = 0; i < E; ++i)
        o.set(i, is_log ? gf[c][i] - row_exp<PRECISE>(yf[c][i]) * sum : yf[c][i] * (gf[c][i] - sum));
      if (j < N) flat_row_store<T, E>(rg, j, N - j, o);
    }
  }
  __syncthreads();
  flat_stage_out<T, BLOCK, U>(gi + row0 * (int64_t)N, bg, nelem);
}

// log_softmax backward for rows beyond what the registers hold of TWO tensors
// (vocabulary-sized rows under cross_entropy): gi = grad - exp(y) * sum(grad).  The
// sum needs grad alone, so grad stays in the registers (V packs a lane on BLOCK
// lanes, in storage format) and y is streamed past it, U packs at a time, the next
// U requested before the current ones are used: every tensor crosses the memory
// interface once, where the multi-pass kernel reads grad twice.  N is a whole
// number of packs and V = ceil(packs / BLOCK) exactly, so only a lane's last pack
// can lie beyond the row end (it is requested from the row's first pack and never
// used) and the others sit at constant strides from the lane's first.
constexpr int kGradResidentUnroll = 4;

template <class TG, class TO, int V, int BLOCK>
__global__ void __launch_bounds__(BLOCK)
log_softmax_bwd_grad_resident_kernel(const TG* __restrict__ grad, const TG* __restrict__ y,
                                     TO* __restrict__ gi, int64_t M, int N) {
  constexpr int E = elems_per_pack<TG>::value;
  constexpr int U = kGradResidentUnroll;
  constexpr bool PRECISE = sizeof(TO) == 4 && sizeof(TG) == 4;
  __shared__ float red[reduce_lds_floats<BLOCK, BLOCK, 1>::value];
  int phase = 0;
  const int lane = threadIdx.x;
  const bool last_in = ((V - 1) * BLOCK + lane) * E < N;  // this lane's last pack lies in the row
  for (int64_t row = blockIdx.x; row < M; row += gridDim.x) {
    const TG* gr = grad + row * (int64_t)N + lane * E;
    const TG* yr = y + row * (int64_t)N + lane * E;
    TO* outr = gi + row * (int64_t)N + lane * E;
    // element offset of pack c from the lane's first pack
    auto off = [&](int c) { return (c < V - 1 || last_in) ? c * BLOCK * E : 0; };
    Pack<TG, E> pg[V], py[U], pn[U];
#pragma unroll
    for (int c = 0; c < V; ++c) pg[c] = Pack<TG, E>::load_stream(gr + off(c));
    auto request_y = [&](int c0, Pack<TG, E> (&dst)[U]) {
#pragma unroll
      for (int u = 0; u < U; ++u)
        if (c0 + u < V) dst[u] = Pack<TG, E>::load_stream(yr + off(c0 + u));
    };
    request_y(0, pn);  // on its way while grad is summed
    float sum[1] = {0.0f};
    if (!last_in) pg[V - 1] = Pack<TG, E>::zero();
#pragma unroll
    for (int c = 0; c < V; ++c)
#pragma unroll
      for (int i = 0; i < E; ++i) sum[0] += pg[c].get(i);
    group_allreduce<BLOCK, BLOCK, 1, SumOp>(sum, red, phase);
    const float s = sum[0];
#pragma unroll
    for (int c0 = 0; c0 < V; c0 += U) {
#pragma unroll
      for (int u = 0; u < U; ++u) py[u] = pn[u];
      if (c0 + U < V) request_y(c0 + U, pn);
#pragma unroll
      for (int u = 0; u < U; ++u) {
        if (c0 + u < V) {
          keep_packed(pg[c0 + u]);
          Pack<TO, E> o;
#pragma unroll
          for (int i = 0; i < E; ++i)
            o.set(i, pg[c0 + u].get(i) - row_exp<PRECISE>(py[u].get(i)) * s);
          if (c0 + u < V - 1 || last_in) o.store_stream(outr + (c0 + u) * BLOCK * E);
        }
      }
    }
  }
}

template <class TG, class TO, int BLOCK, bool MASKED>
__global__ void __launch_bounds__(BLOCK)
softmax_bwd_stream_kernel(const TG* __restrict__ grad, const TG* __restrict__ y,
                          TO* __restrict__ gi, MaskRef mask, int64_t M, int N, int flags) {
  constexpr int E = elems_per_pack<TG>::value;
  constexpr int U = kStreamUnroll;
  constexpr bool PRECISE = sizeof(TO) == 4 && sizeof(TG) == 4;
  constexpr bool WINDOW = softmax_row_window<TG>();
  __shared__ float red[reduce_lds_floats<BLOCK, BLOCK, 1>::value];
  int phase = 0;
  const bool is_log = (flags & kSoftmaxLog) != 0;
  const bool y_whole = WINDOW && same_pack_alignment(grad, y);
  // a pack of y: whole when it is aligned like grad's, else element by element at the row ends
  auto load_y = [&](const TG* yr, int e0, int nw, bool in_row, int h, auto stream_tag) {
    constexpr bool STREAM = decltype(stream_tag)::value;
    return y_whole ? load_window_pack<TG, E, STREAM>(yr, e0, nw, in_row, 0.0f)
                   : load_row_pack<TG, E, STREAM>(yr, e0, nw, in_row, 0.0f, h);
  };
  for (int64_t row = blockIdx.x; row < M; row += gridDim.x) {
    // 16-bit rows: the 16-byte aligned window that holds the row of grad, elements [h, nw) of it
    const int h = WINDOW ? window_head<TG, E>(grad + row * (int64_t)N) : 0;
    const int nw = N + h;
    const int npacks = (nw + E - 1) / E;
    const TG* gr = grad + row * (int64_t)N - h;
    const TG* yr = y + row * (int64_t)N - h;
    TO* outr = gi + row * (int64_t)N - h;
    const uint8_t* mrow = MASKED ? mask_row_ptr(mask, row, N) - h : nullptr;
    auto saved_output = [&](const Pack<TG, E>& p, const Pack<uint8_t, E>& mk, int i) {
      const float v = p.get(i);
      if constexpr (MASKED) return mk.v[i] ? 0.0f : v;
      return v;
    };
    // first pass: sum(grad) for log_softmax (y is not read), sum(y * grad) otherwise
    float sum[1] = {0.0f};
    for (int pk0 = threadIdx.x; pk0 < npacks; pk0 += U * BLOCK) {
      Pack<TG, E> pg[U], py[U];
      Pack<uint8_t, E> mk[U];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int pk = pk0 + u * BLOCK;
        pg[u] = stream_load<TG, E, false, WINDOW>(gr, pk * E, nw, pk < npacks, 0.0f, h);
        if (!is_log) {
          py[u] = load_y(yr, pk * E, nw, pk < npacks, h, std::false_type{});
          if constexpr (MASKED) mk[u] = load_mask_pack<E, false>(mrow, pk * E, nw, pk < npacks, h);
        }
      }
#pragma unroll
      for (int u = 0; u < U; ++u) {
        if constexpr (WINDOW) trim_window_pack<TG, E>(pg[u], (pk0 + u * BLOCK) * E, nw, 0.0f, h);
        if (!is_log && y_whole) trim_window_pack<TG, E>(py[u], (pk0 + u * BLOCK) * E, nw, 0.0f, h);
        if (is_log) {
          ROWNORM_UNIFORM_ARM("log_softmax backward: sum of grad");
#pragma unroll
          for (int i = 0; i < E; ++i) sum[0] += pg[u].get(i);
        } else {
          ROWNORM_UNIFORM_ARM("softmax backward: sum of y * grad");
#pragma unroll
          for (int i = 0; i < E; ++i)
            sum[0] = fmaf(saved_output(py[u], mk[u], i), pg[u].get(i), sum[0]);
        }
      }
    }
    group_allreduce<BLOCK, BLOCK, 1, SumOp>(sum, red, phase);
    const float s = sum[0];
    for (int pk0 = threadIdx.x; pk0 < npacks; pk0 += U * BLOCK) {
      Pack<TG, E> pg[U], py[U];
      Pack<uint8_t, E> mk[U];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int pk = pk0 + u * BLOCK;
        pg[u] = stream_load<TG, E, true, WINDOW>(gr, pk * E, nw, pk < npacks, 0.0f, h);
        py[u] = load_y(yr, pk * E, nw, pk < npacks, h, std::true_type{});
        if constexpr (MASKED) mk[u] = load_mask_pack<E, false>(mrow, pk * E, nw, pk < npacks, h);
      }
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int pk = pk0 + u * BLOCK;
        Pack<TO, E> o;
        if (is_log) {
          ROWNORM_UNIFORM_ARM("log_softmax backward");
#pragma unroll
          for (int i = 0; i < E; ++i)
            o.set(i, pg[u].get(i) - row_exp<PRECISE>(saved_output(py[u], mk[u], i)) * s);
        } else {
          ROWNORM_UNIFORM_ARM("softmax backward");
#pragma unroll
          for (int i = 0; i < E; ++i)
            o.set(i, saved_output(py[u], mk[u], i) * (pg[u].get(i) - s));
        }
        store_row_pack<TO, E, true>(outr, pk * E, nw, pk < npacks, o, h);
      }
    }
  }
}

// ---------------------------------------------------------------------------
// Backward for the rows softmax_fwd_team_kernel serves: a team of workgroups holds a row
// of grad and y in registers (V packs a lane of each, up to 8), each workgroup publishes
// its chunk's sum -- of y * grad, or of grad for log_softmax --, the team's sums are added
// in chunk order, and each workgroup writes its chunk of the gradient out of its
// registers.  grad and y are read once.  A workgroup whose wait runs out sums the whole
// row itself (gi must not overlap grad or y) and loads its chunk again.
template <class TG, class TO, int V>
__global__ void __launch_bounds__(kTeamBlock, kTeamPerCu * kTeamBlock / 256)
softmax_bwd_team_kernel(const TG* __restrict__ grad, const TG* __restrict__ y, TO* __restrict__ gi,
                        int64_t M, int N, int flags, int team, int64_t chunk_packs, TeamSlot* slot,
                        unsigned int call_id, unsigned long long wait_ticks) {
  constexpr int E = elems_per_pack<TG>::value;
  constexpr int BLOCK = kTeamBlock;
  constexpr bool PRECISE = sizeof(TO) == 4 && sizeof(TG) == 4;
  __shared__ float red[reduce_lds_floats<BLOCK, BLOCK, 1>::value];
  __shared__ double tpart[kTeamMaxWorkgroups][2];
  __shared__ float stat[4];  // the row's sum, -, -, whether the team failed
  int phase = 0;
  const bool is_log = (flags & kSoftmaxLog) != 0;
  const int tm = (int)blockIdx.x / team;
  const int c = (int)blockIdx.x - tm * team;
  const int teams = (int)gridDim.x / team;
  const int npacks = N / E;
  const int64_t p0 = (int64_t)c * chunk_packs;
  const int64_t p1 = p0 + chunk_packs < npacks ? p0 + chunk_packs : npacks;
  const int nloc = p1 > p0 ? (int)(p1 - p0) : 0;  // packs of this chunk
  const bool full = nloc == V * BLOCK;  // (uniform) all chunks but a row's last
  const int64_t pbase = nloc > 0 ? p0 : 0;
  const uint32_t loff = (uint32_t)(threadIdx.x * 16);
  const uint32_t ooff = (uint32_t)(threadIdx.x * E * sizeof(TO));
  // (a pointer into global memory, as in the forward)
  auto at = [](auto* p, uint32_t off) {
    using Elem = std::remove_pointer_t<decltype(p)>;
    typedef __attribute__((address_space(1))) Elem* GlobalPtr;
    return (Elem*)reinterpret_cast<GlobalPtr>(reinterpret_cast<uintptr_t>(p) + off);
  };
  unsigned int round = 0;
  for (int64_t row = tm; row < M; row += teams, ++round) {
    TeamEntry* entries = slot->entry[round & 1u];
    if (threadIdx.x == 0) team_store(&entries[blockIdx.x].tag, 0ull);
    const TG* gr = grad + row * (int64_t)N;
    const TG* yr = y + row * (int64_t)N;
    const TG* gb = gr + pbase * E;
    const TG* yb = yr + pbase * E;
    Pack<TG, E> gp[V], yp[V];
    auto load_chunk = [&]() {
      if (full) {
        // (straight-line code: 2 V requests in flight a lane, nothing conditional)
#pragma unroll
        for (int k = 0; k < V; ++k) {
          gp[k] = Pack<TG, E>::load_stream(at(gb + k * BLOCK * E, loff));
          yp[k] = Pack<TG, E>::load_stream(at(yb + k * BLOCK * E, loff));
        }
      } else {
#pragma unroll
        for (int k = 0; k < V; ++k) {
          gp[k] = Pack<TG, E>::zero();
          yp[k] = Pack<TG, E>::zero();
          if (k * BLOCK + (int)threadIdx.x < nloc) {
            gp[k] = Pack<TG, E>::load_stream(at(gb + k * BLOCK * E, loff));
            yp[k] = Pack<TG, E>::load_stream(at(yb + k * BLOCK * E, loff));
          }
        }
      }
    };
    load_chunk();
    float sum[1] = {0.0f};
    if (is_log) {
      ROWNORM_UNIFORM_ARM("log_softmax backward: sum of grad");
#pragma unroll
      for (int k = 0; k < V; ++k) {
#pragma unroll
        for (int i = 0; i < E; ++i) sum[0] += gp[k].get(i);
        __builtin_amdgcn_sched_barrier(0);  // (one pack widened at a time: registers)
      }
    } else {
      ROWNORM_UNIFORM_ARM("softmax backward: sum of y * grad");
#pragma unroll
      for (int k = 0; k < V; ++k) {
#pragma unroll
        for (int i = 0; i < E; ++i) sum[0] = fmaf(yp[k].get(i), gp[k].get(i), sum[0]);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    // (the chunk stays in storage format across the reduction and the wait)
#pragma unroll
    for (int k = 0; k < V; ++k) {
      keep_packed(gp[k]);
      keep_packed(yp[k]);
    }
    group_allreduce<BLOCK, BLOCK, 1, SumOp>(sum, red, phase);
    if (threadIdx.x < 64) {  // the first wavefront publishes, waits and adds up
      const int lane = (int)threadIdx.x;
      const bool complete = team_publish_and_gather(slot, entries, tm, team, call_id, round,
                                                    wait_ticks, (double)sum[0], 0.0, tpart);
      // (the lanes of a wavefront see one another's LDS stores in program order)
      if (complete) {
        float ss = 0.0f;
        for (int j = lane; j < team; j += 64) ss += (float)tpart[j][0];
        ss = wave_group_allreduce<64, SumOp>(ss);
        if (lane == 0) {
          stat[0] = ss;
          stat[3] = 0.0f;
        }
      } else if (lane == 0) {
        stat[3] = 1.0f;
      }
    }
    __syncthreads();
    if (stat[3] != 0.0f) {  // (uniform over the workgroup)
      // The team did not come together: the sum over the whole row, then the chunk again.
      float ws[1] = {0.0f};
      for (int pk0 = threadIdx.x; pk0 < npacks; pk0 += kStreamUnroll * BLOCK) {
        Pack<TG, E> pg[kStreamUnroll], py[kStreamUnroll];
#pragma unroll
        for (int u = 0; u < kStreamUnroll; ++u) {
          const int pk = pk0 + u * BLOCK;
          pg[u] = Pack<TG, E>::zero();
          py[u] = Pack<TG, E>::zero();
          if (pk < npacks) {
            pg[u] = Pack<TG, E>::load(gr + (int64_t)pk * E);
            if (!is_log) py[u] = Pack<TG, E>::load(yr + (int64_t)pk * E);
          }
        }
#pragma unroll
        for (int u = 0; u < kStreamUnroll; ++u)
#pragma unroll
          for (int i = 0; i < E; ++i)
            ws[0] = is_log ? ws[0] + pg[u].get(i) : fmaf(py[u].get(i), pg[u].get(i), ws[0]);
      }
      group_allreduce<BLOCK, BLOCK, 1, SumOp>(ws, red, phase);
      if (threadIdx.x == 0) stat[0] = ws[0];
      __syncthreads();
      load_chunk();
    }
    const float s = stat[0];
    TO* ob = gi + row * (int64_t)N + pbase * E;
#pragma unroll
    for (int k = 0; k < V; ++k) {
      if (full || k * BLOCK + (int)threadIdx.x < nloc) {
        Pack<TO, E> o;
        if (is_log) {
          ROWNORM_UNIFORM_ARM("log_softmax backward");
#pragma unroll
          for (int i = 0; i < E; ++i) o.set(i, gp[k].get(i) - row_exp<PRECISE>(yp[k].get(i)) * s);
        } else {
          ROWNORM_UNIFORM_ARM("softmax backward");
#pragma unroll
          for (int i = 0; i < E; ++i) o.set(i, yp[k].get(i) * (gp[k].get(i) - s));
        }
        o.store_stream(at(ob + k * BLOCK * E, ooff));
      }
      // (pack k + 1 is widened after pack k has been stored, not before: registers)
      __builtin_amdgcn_sched_barrier(0);
    }
    // stat[] is rewritten for the next row only after every thread has passed the
    // barrier of the next block reduction, i.e. after it has read this row's value
  }
}

}  // namespace rownorm
