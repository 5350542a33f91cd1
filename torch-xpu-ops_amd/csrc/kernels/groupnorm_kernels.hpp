// GroupNorm forward and backward kernels for gfx950 (wave64), NCHW-contiguous input.
//
// X is [N, C, HxW]; with `groups` groups of D = C / groups channels each, the
// (n, g) slab of L = D * HxW contiguous elements is one row of a dense
// [N * groups, L] matrix, normalized like a LayerNorm row, and the affine
// weights are per channel: element p of row (n, g) uses channel g * D + p / HxW.
// The row layout is that of the LayerNorm kernels (G lanes share a row, V
// 16-byte packs per lane, BLOCK / G rows per workgroup), so X is read once and
// Y written once; the backward reads dY and X once, writes dX once and leaves
// the per-(n, channel) sums of dY * xhat and dY in an fp32 [N, C] workspace that
// colsum_finalize_kernel adds up over n.
//
// Three kinds of resident kernel (MODE):
//   kGnUniform   HxW is a whole number of packs, so every pack lies in one
//                channel: one weight lookup per pack, branch-free row access,
//                channel sums fused into the backward through an LDS staging area.
//   kGnStraddle  rows are whole packs (L % E == 0) but channels are not (7x7 and
//                14x14 feature maps in 16 bits): a pack lies in one channel or
//                straddles the border of two, so it looks up two weights and each
//                element selects; row access and the fused channel sums as above,
//                the part of a straddling pack that belongs to the next channel
//                travels through a small LDS array of its own.
//   kGnGeneral   anything else: the channel is looked up per element, row access
//                is the general one, and the channel sums come from
//                gn_channel_sums_kernel, which reads dY and X a second time.
// Rows too long for the registers: the forward takes two passes over the row; the
// backward computes the channel sums first and dX from them, element by element.
//
// What these stand in for in the reference (src/ATen/native/xpu/sycl/
// GroupNormKernels.cpp): GNRowwiseMomentsFunctor / ...VectorizedFunctor
// (:72-218) + ComputeFusedParamsFunctor (:220-260) + the elementwise
// GroupNormFunctor pass (:351-357, :446-496), three launches that read X
// twice; and for the backward ComputeInternalGradients[Vectorized]Functor
// (:943-1072), ComputeBackwardFusedParamsFunctor (:1088-1165), the elementwise
// dX pass (:1081-1086, :1476-1520) and GammaBetaBackward[Plain]Functor
// (:1167-1351), which read dY and X twice.  Formulas (same file):
//   y  = (x - mean) * rstd * gamma[c] + beta[c]
//   ds[n,c] = sum_hw dy * x,  db[n,c] = sum_hw dy                       (:955-975)
//   dx = rstd*gamma[c]*dy + c2*x + c3 with
//        c2 = (sum_c db*gamma * mean - sum_c ds*gamma) * rstd^3 / L,
//        c3 = -c2 * mean - sum_c db*gamma * rstd / L                    (:1133-1160)
//   dgamma[c] = sum_n (ds - db * mean) * rstd,  dbeta[c] = sum_n db     (:1195-1215)
// Here dx is evaluated in the equivalent LayerNorm form
//   dx = (rstd / L) * (L * g - xhat * s2 - s1),  g = dy * gamma[c],
//   s1 = sum g, s2 = sum g * xhat, xhat = (x - mean) * rstd,
// which does not cancel when mean is large against the spread.
//
// mean and rstd are stored in the weight dtype WT (the row dtype when the
// weights share it, fp32 beside fp32 weights), as native_group_norm returns them.
#pragma once
#include <type_traits>

#include "device/pack.hpp"
#include "device/reduce.hpp"
#include "device/team.hpp"
#include "plan.hpp"

namespace rownorm {

struct GroupShape {
  int L;        // elements per (n, g) row: D * HxW
  int HxW;      // elements per channel
  int D;        // channels per group
  int groups;   // groups per sample
  // rows whose channels are whole packs (HxW % E == 0), else both 0:
  int packs;            // packs per row, L / E
  unsigned pack_magic;  // ceil(2^31 / (HxW / E)), see gn_pack_channel
  // rows of whole packs whose channels are not (kGnStraddle), else 0:
  unsigned elem_magic;  // ceil(2^32 / HxW), see gn_straddle
};



// Wavefronts per SIMD a resident kernel is compiled for (the second argument of
// __launch_bounds__): the 512-lane layouts with 6 packs or more that the
// planner prefers to 1024 lanes must leave room for two workgroups a compute
// unit, i.e. 4 wavefronts per SIMD, 128 VGPRs a lane.
constexpr int gn_min_waves(int G, int V, int max_v) {
  return (G == 512 && V > 5 && V <= max_v) ? 4 : 1;
}

// Channel (index into gamma/beta) of element p of row `g` (p is clamped into the row).
__device__ __forceinline__ int gn_channel(const GroupShape& s, int g, int p) {
  const int pc = p < s.L ? p : s.L - 1;
  return g * s.D + (int)((unsigned)pc / (unsigned)s.HxW);
}

// Channel of pack `pk` of row `g` when every pack lies in one channel (pk is
// clamped into the row).  pk / S for S = HxW / E packs per channel is
// floor(2 * pk * ceil(2^31 / S) / 2^32), exact while pk * S < 2^31; the rows
// held in registers have at most 2^14 packs.  A 32-bit division costs about
// 25 instructions a pack, this costs 3.
__device__ __forceinline__ int gn_pack_channel(const GroupShape& s, int g, int pk) {
  const int pc = pk < s.packs ? pk : s.packs - 1;
  return g * s.D + (int)__umulhi(2u * (unsigned)pc, s.pack_magic);
}

// Where the pack at element e0 of a row lies among the channels when channels
// are not whole packs: `ch` = channel (within the group) of its first element,
// `bnd` = how many of its elements belong to that channel (>= E: all of them;
// the others belong to channel ch + 1).  HxW >= E, so a pack meets one border
// at most.  e0 / HxW is floor(e0 * ceil(2^32 / HxW) / 2^32), exact while
// e0 * HxW < 2^32, and a register-resident row has at most 2^16 elements.
struct GnStraddle {
  int ch, bnd;
};
__device__ __forceinline__ GnStraddle gn_straddle(const GroupShape& s, int e0, int E) {
  const int ec = e0 < s.L ? e0 : s.L - E;  // packs past the row end: any pack of the row
  GnStraddle r;
  r.ch = (int)__umulhi((unsigned)ec, s.elem_magic);
  r.bnd = (r.ch + 1) * s.HxW - ec;
  return r;
}

template <class WT>
__device__ __forceinline__ float gn_weight(const WT* w, int ch, float dflt) {
  return w ? (float)w[(unsigned)ch] : dflt;  // ch >= 0: a 32-bit offset from a scalar base
}
// The same when the caller knows whether the weight exists (HAVE): with it, a plain
// load.  The test of the pointer above is a branch around the load, and the join of
// a branch waits for every request outstanding, so lookups that go through it
// complete one after the other, each behind whatever was stored before it.
template <bool HAVE, class WT>
__device__ __forceinline__ float gn_weight_known(const WT* w, int ch, float dflt) {
  if constexpr (HAVE)
    return (float)w[(unsigned)ch];
  else
    return gn_weight(w, ch, dflt);
}

// ---------------------------------------------------------------------------
// Forward, row resident in registers.  Statistics as in the LayerNorm kernel:
// a centre mean0, centred sums over the registers, mean = mean0 + s1/L,
// var = (s2 - s1*s1/L)/L; y uses (x - mean0) - s1/L so that a constant row
// gives beta bit for bit.
template <class T, class WT, int G, int V, int BLOCK, int MODE>
__global__ void __launch_bounds__(BLOCK, gn_min_waves(G, V, group_half_lanes_max_v(OC_GROUP_FWD)))
gn_fwd_resident_kernel(const T* __restrict__ x, const WT* __restrict__ gamma,
                       const WT* __restrict__ beta, T* __restrict__ y, WT* __restrict__ mean,
                       WT* __restrict__ rstd, int64_t rows, GroupShape s, float eps) {
  constexpr int E = elems_per_pack<T>::value;
  constexpr int RPB = BLOCK / G;
  constexpr bool UNIFORM = MODE != kGnGeneral;  // rows of whole packs: branch-free row access
  constexpr bool STRADDLE = MODE == kGnStraddle;
  __shared__ float red[reduce_lds_floats<G, BLOCK, 2>::value];
  int phase = 0;
  const int slot = threadIdx.x / G;
  const int lane0 = threadIdx.x % G;
  const float fL = (float)s.L;
  const float inv_l = 1.0f / fL;
  const bool exact = s.L == G * V * E;
  const int64_t nrb = (rows + RPB - 1) / RPB;
  for (int64_t rb = blockIdx.x; rb < nrb; rb += gridDim.x) {
    // opaque once a row, so that the V packs' offsets and channels are computed
    // where they are used instead of being held in registers across the loop
    // (see the backward)
    int lane = lane0;
    asm volatile("" : "+v"(lane));
    const int64_t row = rb * RPB + slot;
    const bool ok = RPB == 1 ? true : row < rows;
    const int64_t rowc = ok ? row : 0;
    const int g = (int)((uint32_t)rowc % (uint32_t)s.groups);
    const T* xr = x + rowc * (int64_t)s.L;
    Pack<T, E> xp[V];
#pragma unroll
    for (int c = 0; c < V; ++c)
      xp[c] = row_load<T, E, true, UNIFORM>(xr, (c * G + lane) * E, s.L, ok, 0.0f);
    // centre of the sums: fp32 rows take the row mean (a reduction round of its
    // own, exact for any data); 16-bit rows take the median of the row's first
    // three elements, which every lane reads for itself, so the statistics need
    // one round (see the LayerNorm forward for the error argument)
    float mean0;
    if constexpr (sizeof(T) == 2) {
      const Pack<T, E> head = load_row_pack<T, E, false>(xr, 0, s.L, true, 0.0f);
      const float a = head.get(0), b = head.get(1), c3 = head.get(2);
      mean0 = fmaxf(fminf(a, b), fminf(fmaxf(a, b), c3));
    } else {
      float acc0[1] = {0.0f};
#pragma unroll
      for (int c = 0; c < V; ++c)
#pragma unroll
        for (int i = 0; i < E; ++i) acc0[0] += xp[c].get(i);
      group_allreduce<G, BLOCK, 1, SumOp>(acc0, red, phase);
      mean0 = acc0[0] / fL;
    }
    float acc[2] = {0.0f, 0.0f};
    auto centred_sums = [&](auto masked) {
      constexpr bool MASKED = decltype(masked)::value;
#pragma unroll
      for (int c = 0; c < V; ++c) {
        keep_packed(xp[c]);
        const int nvalid = ok ? s.L - (c * G + lane) * E : 0;
#pragma unroll
        for (int i = 0; i < E; ++i) {
          float d = xp[c].get(i) - mean0;
          if constexpr (MASKED) d = (i < nvalid) ? d : 0.0f;
          acc[0] += d;
          acc[1] = fmaf(d, d, acc[1]);
        }
      }
    };
    if (exact)
      centred_sums(std::false_type{});
    else
      centred_sums(std::true_type{});
    group_allreduce<G, BLOCK, 2, SumOp>(acc, red, phase);
    const float m1 = row_mean_of<T>(acc[0], fL, inv_l);
    float var = row_mean_of<T>(acc[1] - acc[0] * m1, fL, inv_l);
    var = var < 0.0f ? 0.0f : var;  // a select, not v_max_f32: a NaN row keeps NaN statistics
    const float rs = row_rstd_of<T>(var + eps);
    T* yr = y + row * (int64_t)s.L;
    if constexpr (UNIFORM) {
      // The weights of pack c + 1 are requested before pack c is normalized and stored:
      // requests complete in order, stores included, so a pack that looked its weights
      // up on its own turn waited for the store of the pack before it.
      struct PackWeights {
        float ga0, ga1, be0, be1;
        int bnd;
      };
      auto normalize = [&](auto have) {
        constexpr bool HAVE = decltype(have)::value;  // gamma and beta both given
        auto lookup = [&](int c) {
          PackWeights w;
          if constexpr (STRADDLE) {
            const GnStraddle sw = gn_straddle(s, (c * G + lane) * E, E);
            const int c0 = g * s.D + sw.ch;
            const int c1 = sw.ch + 1 < s.D ? c0 + 1 : c0;
            w.ga0 = gn_weight_known<HAVE>(gamma, c0, 1.0f);
            w.ga1 = gn_weight_known<HAVE>(gamma, c1, 1.0f);
            w.be0 = gn_weight_known<HAVE>(beta, c0, 0.0f);
            w.be1 = gn_weight_known<HAVE>(beta, c1, 0.0f);
            w.bnd = sw.bnd;
          } else {
            const int ch = gn_pack_channel(s, g, c * G + lane);
            w.ga0 = w.ga1 = gn_weight_known<HAVE>(gamma, ch, 1.0f);
            w.be0 = w.be1 = gn_weight_known<HAVE>(beta, ch, 0.0f);
            w.bnd = E;
          }
          return w;
        };
        PackWeights wn = lookup(0);
#pragma unroll
        for (int c = 0; c < V; ++c) {
          const PackWeights w = wn;
          if (c + 1 < V) wn = lookup(c + 1);
          __builtin_amdgcn_sched_barrier(0);
          keep_packed(xp[c]);
          const float ga0 = w.ga0 * rs, ga1 = w.ga1 * rs;
          Pack<T, E> o;
#pragma unroll
          for (int i = 0; i < E; ++i) {
            const bool first = !STRADDLE || i < w.bnd;
            o.set(i,
                  ((xp[c].get(i) - mean0) - m1) * (first ? ga0 : ga1) + (first ? w.be0 : w.be1));
          }
          row_store<T, E, true, UNIFORM>(yr, (c * G + lane) * E, s.L, ok, o);
          __builtin_amdgcn_sched_barrier(0);
        }
      };
      if (gamma != nullptr && beta != nullptr)
        normalize(std::true_type{});
      else
        normalize(std::false_type{});
    } else {
#pragma unroll
      for (int c = 0; c < V; ++c) {
        keep_packed(xp[c]);
        const int e0 = (c * G + lane) * E;
        Pack<T, E> o;
#pragma unroll
        for (int i = 0; i < E; ++i) {
          const int ch = gn_channel(s, g, e0 + i);
          const float ga = gn_weight(gamma, ch, 1.0f) * rs;
          o.set(i, ((xp[c].get(i) - mean0) - m1) * ga + gn_weight(beta, ch, 0.0f));
        }
        row_store<T, E, true, UNIFORM>(yr, e0, s.L, ok, o);
      }
    }
    if (ok && lane == 0) {
      if (mean) mean[row] = (WT)(rs == rs ? mean0 + m1 : rs);  // NaN variance: NaN mean
      if (rstd) rstd[row] = (WT)rs;
    }
  }
}

// ---------------------------------------------------------------------------
// The same forward for 16-bit rows that fill a layout of whole wavefronts exactly
// (L == G * V * E, one row a workgroup) and whose channels are whole runs of 64
// packs (HxW / E a multiple of 64, a diffusion UNet's 64x64 and 32x32 maps): the
// 64 packs a wavefront moves with one instruction lie in one channel, so a
// channel's weights are two scalar loads, the row pointer is scalar arithmetic, the
// head of the row (the centre of the sums) is a scalar load, and no access is
// conditional.  Arithmetic is that of gn_fwd_resident_kernel for the same layout,
// bit for bit.  Measured on one MI355X, bf16 [64, 320, 64, 64] with 32 groups (2048
// rows of 40960 elements on 512 lanes x 10 packs, two workgroups a compute unit):
// 61.6 -> 58.6 us.  Requesting the next row ahead of the current one (a second and
// third register set) measured the same or slower at every layout tried.
template <class T, class WT, int G, int V>
__global__ void __launch_bounds__(G)
gn_fwd_exact_kernel(const T* __restrict__ x, const WT* __restrict__ gamma,
                    const WT* __restrict__ beta, T* __restrict__ y, WT* __restrict__ mean,
                    WT* __restrict__ rstd, int64_t rows, GroupShape s, float eps) {
  constexpr int E = elems_per_pack<T>::value;
  static_assert(sizeof(T) == 2 && G % 64 == 0, "16-bit rows on whole wavefronts");
  __shared__ float red[reduce_lds_floats<G, G, 2>::value];
  int phase = 0;
  const float fL = (float)s.L;
  const float inv_l = 1.0f / fL;
  const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
  const unsigned S = (unsigned)(s.HxW / E);  // packs per channel
  int chl[V];                                // channel (within the group) of pack c
#pragma unroll
  for (int c = 0; c < V; ++c) chl[c] = (int)((unsigned)(c * G + wave * 64) / S);
  const uint32_t loff = (uint32_t)(threadIdx.x * E * (int)sizeof(T));
  auto at = [](const T* p, uint32_t off) {
    return reinterpret_cast<const T*>(reinterpret_cast<const char*>(p) + off);
  };
  // absent weights: the loads go to memory that exists and their values are not used
  const bool has_g = gamma != nullptr, has_b = beta != nullptr;
  const WT* gsrc = has_g ? gamma : reinterpret_cast<const WT*>(x);
  const WT* bsrc = has_b ? beta : reinterpret_cast<const WT*>(x);
  for (int64_t row = blockIdx.x; row < rows; row += gridDim.x) {
    const int ch0 = (int)((uint32_t)row % (uint32_t)s.groups) * s.D;
    const T* xr = x + row * (int64_t)s.L;
    const uint64_t head = uniform_load<uint64_t>(xr);
    UniformElem<WT> wg[V], wb[V];
    Pack<T, E> xp[V];
#pragma unroll
    for (int c = 0; c < V; ++c) {
      wg[c] = UniformElem<WT>::load(gsrc, ch0 + chl[c]);
      wb[c] = UniformElem<WT>::load(bsrc, ch0 + chl[c]);
      xp[c] = Pack<T, E>::load_stream(at(xr + c * G * E, loff));
    }
    const float a = (float)__builtin_bit_cast(T, (uint16_t)head);
    const float b = (float)__builtin_bit_cast(T, (uint16_t)(head >> 16));
    const float c3 = (float)__builtin_bit_cast(T, (uint16_t)(head >> 32));
    const float mean0 = fmaxf(fminf(a, b), fminf(fmaxf(a, b), c3));
    float acc[2] = {0.0f, 0.0f};
#pragma unroll
    for (int c = 0; c < V; ++c) {
      keep_packed(xp[c]);
#pragma unroll
      for (int i = 0; i < E; ++i) {
        const float d = xp[c].get(i) - mean0;
        acc[0] += d;
        acc[1] = fmaf(d, d, acc[1]);
      }
    }
    group_allreduce<G, G, 2, SumOp>(acc, red, phase);
    const float m1 = row_mean_of<T>(acc[0], fL, inv_l);
    float var = row_mean_of<T>(acc[1] - acc[0] * m1, fL, inv_l);
    var = var < 0.0f ? 0.0f : var;  // a select: a NaN row keeps NaN statistics
    const float rs = row_rstd_of<T>(var + eps);
    if (threadIdx.x == 0) {
      if (mean) mean[row] = (WT)(rs == rs ? mean0 + m1 : rs);  // NaN variance: NaN mean
      if (rstd) rstd[row] = (WT)rs;
    }
    T* yr = y + row * (int64_t)s.L;
#pragma unroll
    for (int c = 0; c < V; ++c) {
      keep_packed(xp[c]);
      const float ga = (has_g ? wg[c].value() : 1.0f) * rs;
      const float be = has_b ? wb[c].value() : 0.0f;
      Pack<T, E> o;
#pragma unroll
      for (int i = 0; i < E; ++i) o.set(i, ((xp[c].get(i) - mean0) - m1) * ga + be);
      o.store_stream(const_cast<T*>(at(yr + c * G * E, loff)));
    }
  }
}

// Forward for rows too long for the registers: one workgroup per row, two
// passes over the row (statistics, normalize).  The statistics are the sums of
// (x - k) and (x - k)^2 in float64, k = the row's first element: float32 and
// 16-bit values and their differences are exact in float64, and with 53-bit
// sums s2 - s1*s1/L keeps its accuracy however far k lies from the row (a zero
// head before a row around 1000 cost rstd 8e-6 with per-thread float32 sums).
// It stands in for the Welford merge of the reference (WelfordOps::combine,
// src/ATen/native/xpu/sycl/SharedReduceOps.h:71-88).  The mean goes to the
// normalize pass as float(mean) plus the remainder, so the rounding of the
// saved statistic never enters y; on a constant row x - k is exactly zero.
template <class T, class WT, int BLOCK>
__global__ void __launch_bounds__(BLOCK)
gn_fwd_stream_kernel(const T* __restrict__ x, const WT* __restrict__ gamma,
                     const WT* __restrict__ beta, T* __restrict__ y, WT* __restrict__ mean,
                     WT* __restrict__ rstd, int64_t rows, GroupShape s, float eps) {
  constexpr int E = elems_per_pack<T>::value;
  __shared__ double red[2 * (BLOCK / 64)];
  __shared__ float stat[3];
  const int npacks = (s.L + E - 1) / E;
  for (int64_t row = blockIdx.x; row < rows; row += gridDim.x) {
    const int g = (int)((uint32_t)row % (uint32_t)s.groups);
    const T* xr = x + row * (int64_t)s.L;
    T* yr = y + row * (int64_t)s.L;
    const double k = (double)(float)xr[0];
    double s1 = 0.0, s2 = 0.0;
    // rows of whole packs: four packs a lane in flight, nothing conditional; the pack
    // sums in float32 about k, their totals in float64 (as add_centred_sums)
    constexpr int U = 4;
    const bool whole = (s.L % E) == 0;  // uniform
    const bool one_weight = (s.HxW % E) == 0 && gamma != nullptr && beta != nullptr;  // uniform
    int pk = threadIdx.x;
    if (whole) {
      const float kf = (float)k;
      for (; pk + (U - 1) * BLOCK < npacks; pk += U * BLOCK) {
        Pack<T, E> p[U];
#pragma unroll
        for (int u = 0; u < U; ++u) p[u] = Pack<T, E>::load(xr + (int64_t)(pk + u * BLOCK) * E);
#pragma unroll
        for (int u = 0; u < U; ++u) {
          if constexpr (sizeof(T) == 2) {
            float t1 = 0.0f, t2 = 0.0f;
#pragma unroll
            for (int i = 0; i < E; ++i) {
              const float d = p[u].get(i) - kf;
              t1 += d;
              t2 = fmaf(d, d, t2);
            }
            s1 += (double)t1;
            s2 += (double)t2;
          } else {
#pragma unroll
            for (int i = 0; i < E; ++i) {
              const double d = (double)p[u].get(i) - k;
              s1 += d;
              s2 = fma(d, d, s2);
            }
          }
        }
      }
    }
    for (; pk < npacks; pk += BLOCK) {
      const Pack<T, E> p = load_row_pack<T, E, false>(xr, pk * E, s.L, true, 0.0f);
      const int nvalid = s.L - pk * E;
#pragma unroll
      for (int i = 0; i < E; ++i) {
        const double d = i < nvalid ? (double)p.get(i) - k : 0.0;
        s1 += d;
        s2 = fma(d, d, s2);
      }
    }
    block_sum2_f64<BLOCK>(s1, s2, red);
    if (threadIdx.x == 0) {
      const double dL = (double)s.L;
      const double m1 = s1 / dL;
      const double mu = k + m1;
      double var = (s2 - s1 * m1) / dL;
      var = var < 0.0 ? 0.0 : var;  // a select: a NaN row keeps NaN statistics
      stat[0] = (float)mu;
      stat[1] = (float)(mu - (double)stat[0]);
      stat[2] = (float)(1.0 / sqrt(var + (double)eps));
    }
    __syncthreads();
    const float hi = stat[0], lo = stat[1], rs = stat[2];
    pk = threadIdx.x;
    if (whole && one_weight) {
      // channels of whole packs as well: one gamma and one beta a pack
      const uint32_t S = (uint32_t)(s.HxW / E);
      for (; pk + (U - 1) * BLOCK < npacks; pk += U * BLOCK) {
        Pack<T, E> p[U];
        WT gw[U], bw[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
          const uint32_t q = (uint32_t)(pk + u * BLOCK);
          p[u] = Pack<T, E>::load_stream(xr + (int64_t)q * E);
          const int ch = g * s.D + (int)(q / S);
          gw[u] = gamma[ch];
          bw[u] = beta[ch];
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
          const float ga = (float)gw[u] * rs, be = (float)bw[u];
          Pack<T, E> o;
#pragma unroll
          for (int i = 0; i < E; ++i) o.set(i, ((p[u].get(i) - hi) - lo) * ga + be);
          o.store_stream(yr + (int64_t)(pk + u * BLOCK) * E);
        }
      }
    }
    for (; pk < npacks; pk += BLOCK) {
      const int e0 = pk * E;
      const Pack<T, E> p = load_row_pack<T, E, true>(xr, e0, s.L, true, 0.0f);
      Pack<T, E> o;
#pragma unroll
      for (int i = 0; i < E; ++i) {
        const int ch = gn_channel(s, g, e0 + i);
        const float ga = gn_weight(gamma, ch, 1.0f) * rs;
        o.set(i, ((p.get(i) - hi) - lo) * ga + gn_weight(beta, ch, 0.0f));
      }
      store_row_pack<T, E, true>(yr, e0, s.L, true, o);
    }
    if (threadIdx.x == 0) {
      if (mean) mean[row] = (WT)(rs == rs ? hi : rs);  // NaN variance: NaN mean
      if (rstd) rstd[row] = (WT)rs;
    }
  }
}

// ---------------------------------------------------------------------------
// Backward, rows resident in registers.  With rows of whole packs and a
// workspace, each lane parks the sums of dy*xhat and dy over each of its packs
// in LDS; after a barrier the channels of the row are summed from there in a
// fixed order (TPC lanes per channel, then a butterfly) and written to part_dg /
// part_db [N, C].  kGnStraddle: a pack parks the sums over its elements of its
// first channel; what a straddling pack holds of the next channel goes to that
// channel's slot of a second array (one straddling pack per channel border, so
// one writer per slot), which the channel's fold adds when the channel does not
// start on a pack.
template <int G, int V, int BLOCK, int MODE>
struct gn_stage_floats {
  static constexpr int value = MODE != kGnGeneral ? 2 * BLOCK * V : 1;
  // per row slot: two floats for each channel the slot's row can have
  static constexpr int next_per_slot =
      MODE == kGnStraddle ? 2 * (G * V < kGnStraddleMaxD ? G * V : kGnStraddleMaxD) : 0;
  static constexpr int next_value = MODE == kGnStraddle ? (BLOCK / G) * next_per_slot : 1;
};

template <class T, class WT, int G, int V, int BLOCK, int MODE>
__global__ void __launch_bounds__(BLOCK, gn_min_waves(G, V, group_half_lanes_max_v(OC_GROUP_BWD)))
gn_bwd_resident_kernel(const T* __restrict__ dy, const T* __restrict__ x,
                       const WT* __restrict__ mean, const WT* __restrict__ rstd,
                       const WT* __restrict__ gamma, T* __restrict__ dx,
                       float* __restrict__ part_dg, float* __restrict__ part_db, int64_t rows,
                       GroupShape s, int tpc_log2) {
  constexpr int E = elems_per_pack<T>::value;
  constexpr int RPB = BLOCK / G;
  constexpr bool UNIFORM = MODE != kGnGeneral;  // rows of whole packs, fused channel sums
  constexpr bool STRADDLE = MODE == kGnStraddle;
  __shared__ float red[reduce_lds_floats<G, BLOCK, 2>::value];
  __shared__ float stage[gn_stage_floats<G, V, BLOCK, MODE>::value];
  __shared__ float stage_next[gn_stage_floats<G, V, BLOCK, MODE>::next_value];
  int phase = 0;
  const int slot = threadIdx.x / G;
  const int lane0 = threadIdx.x % G;
  const float fL = (float)s.L;
  const bool want_cols = UNIFORM && part_dg != nullptr;  // uniform over the grid
  const int64_t nrb = (rows + RPB - 1) / RPB;
  for (int64_t rb = blockIdx.x; rb < nrb; rb += gridDim.x) {
    // The lane index is made opaque once a row: the offsets, channels and LDS
    // slots of the V packs derive from it, and the compiler would otherwise
    // compute all of them before the loop and hold 3-4 registers a pack for the
    // whole kernel (spilling at 7 and 8 packs).  Recomputing costs a few
    // instructions a pack.
    int lane = lane0;
    asm volatile("" : "+v"(lane));
    const int64_t row = rb * RPB + slot;
    const bool ok = RPB == 1 ? true : row < rows;
    const int64_t rowc = ok ? row : 0;
    const int g = (int)((uint32_t)rowc % (uint32_t)s.groups);
    const float mu = (float)mean[rowc];
    const float rs = (float)rstd[rowc];
    Pack<T, E> xp[V], dp[V];
#pragma unroll
    for (int c = 0; c < V; ++c) {
      const int e0 = (c * G + lane) * E;
      xp[c] = row_load<T, E, true, UNIFORM>(x + rowc * (int64_t)s.L, e0, s.L, ok, 0.0f);
      dp[c] = row_load<T, E, true, UNIFORM>(dy + rowc * (int64_t)s.L, e0, s.L, ok, 0.0f);
    }
    float acc[2] = {0.0f, 0.0f};
    float gu[UNIFORM ? V : 1];  // the weight of each pack, looked up once a row
    float gv[STRADDLE ? V : 1];  // kGnStraddle: the weight of the pack's second channel
    int bnd[STRADDLE ? V : 1];   //              and the elements that belong to the first
    float* st = stage + slot * (UNIFORM ? 2 * G * V : 0);
    float* sn = stage_next + slot * gn_stage_floats<G, V, BLOCK, MODE>::next_per_slot;
    // (one copy of the loop per case of gamma: see gn_weight_known)
    auto row_sums = [&](auto have) {
      constexpr bool HAVE = decltype(have)::value;
#pragma unroll
      for (int c = 0; c < V; ++c) {
        const int e0 = (c * G + lane) * E;
        if constexpr (STRADDLE) {
          const GnStraddle w = gn_straddle(s, e0, E);
          const bool has_next = w.bnd < E && w.ch + 1 < s.D;
          const float ga = gu[c] = gn_weight_known<HAVE>(gamma, g * s.D + w.ch, 1.0f);
          const float gb = gv[c] = gn_weight_known<HAVE>(gamma, g * s.D + (has_next ? w.ch + 1 : w.ch), 1.0f);
          bnd[c] = w.bnd;
          float pdg = 0.0f, pdb = 0.0f, fdg = 0.0f, fdb = 0.0f;  // whole pack / first channel
#pragma unroll
          for (int i = 0; i < E; ++i) {
            const float gy = dp[c].get(i);
            const float t = gy * (xp[c].get(i) - mu);
            pdb += gy;
            pdg += t;
            fdb += i < w.bnd ? gy : 0.0f;
            fdg += i < w.bnd ? t : 0.0f;
          }
          // (a pack that lies in one channel adds the same terms to both pairs: the
          // second channel's share is then exactly zero)
          const float ndg = pdg - fdg, ndb = pdb - fdb;
          acc[0] = fmaf(fdb, ga, fmaf(ndb, gb, acc[0]));
          acc[1] = fmaf(fdg * rs, ga, fmaf(ndg * rs, gb, acc[1]));
          if (want_cols) {
            st[2 * (c * G + lane)] = fdg * rs;
            st[2 * (c * G + lane) + 1] = fdb;
            if (has_next && e0 < s.L) {
              sn[2 * (w.ch + 1)] = ndg * rs;
              sn[2 * (w.ch + 1) + 1] = ndb;
            }
          }
        } else if constexpr (UNIFORM) {
          const float ga = gu[c] = gn_weight_known<HAVE>(gamma, gn_pack_channel(s, g, c * G + lane), 1.0f);
          float pdg = 0.0f, pdb = 0.0f;
#pragma unroll
          for (int i = 0; i < E; ++i) {
            const float gy = dp[c].get(i);
            pdb += gy;
            pdg = fmaf(gy, xp[c].get(i) - mu, pdg);
          }
          // zero-filled packs (row slot or pack out of range) add nothing
          acc[0] = fmaf(pdb, ga, acc[0]);
          acc[1] = fmaf(pdg * rs, ga, acc[1]);
          if (want_cols) {
            st[2 * (c * G + lane)] = pdg * rs;
            st[2 * (c * G + lane) + 1] = pdb;
          }
        } else {
#pragma unroll
          for (int i = 0; i < E; ++i) {
            const float ga = gn_weight_known<HAVE>(gamma, gn_channel(s, g, e0 + i), 1.0f);
            const float gv = dp[c].get(i) * ga;
            acc[0] += gv;
            acc[1] = fmaf(gv, (xp[c].get(i) - mu) * rs, acc[1]);
          }
        }
      }
    };
    if (gamma != nullptr)
      row_sums(std::true_type{});
    else
      row_sums(std::false_type{});
    group_allreduce<G, BLOCK, 2, SumOp>(acc, red, phase);
    if (dx != nullptr) {
      T* dr = dx + row * (int64_t)s.L;
      const float s1 = acc[0], s2 = acc[1];
      const float term1 = rs / fL;
      // 16-bit rows with one weight a pack use the regrouped
      // dy*(rs*gamma) - x*(rs*a) + (mu*rs*a - b), a = s2*rs/L, b = s1*rs/L: two
      // FMAs an element, rounding far below a 16-bit ulp (as the LayerNorm backward)
      const float ra = rs * (s2 * term1);
      const float cc = mu * ra - s1 * term1;
#pragma unroll
      for (int c = 0; c < V; ++c) {
        keep_packed(xp[c]);
        keep_packed(dp[c]);
        const int e0 = (c * G + lane) * E;
        const float gr = UNIFORM ? gu[c] * rs : 0.0f;
        const float gq = STRADDLE ? gv[c] * rs : 0.0f;
        Pack<T, E> o;
#pragma unroll
        for (int i = 0; i < E; ++i) {
          if constexpr (UNIFORM && sizeof(T) == 2) {
            const float gri = STRADDLE ? (i < bnd[c] ? gr : gq) : gr;
            o.set(i, fmaf(xp[c].get(i), -ra, fmaf(dp[c].get(i), gri, cc)));
          } else {
            const float ga = STRADDLE ? (i < bnd[c] ? gu[c] : gv[c])
                             : UNIFORM ? gu[c]
                                       : gn_weight(gamma, gn_channel(s, g, e0 + i), 1.0f);
            const float xh = (xp[c].get(i) - mu) * rs;
            float f = fL * (dp[c].get(i) * ga);
            f -= xh * s2;
            f -= s1;
            o.set(i, f * term1);
          }
        }
        row_store<T, E, true, UNIFORM>(dr, e0, s.L, ok, o);
      }
    }
    if constexpr (UNIFORM) {
      if (want_cols) {
        __syncthreads();
        // channel d of the row owns packs [d * S, (d + 1) * S), S = HxW / E; with
        // straddling packs, the packs whose first element lies in it:
        // [ceil(d * HxW / E), ceil((d + 1) * HxW / E))
        const int S = s.HxW / E;
        const int TPC = 1 << tpc_log2;  // lanes per channel, power of two <= min(G, 64)
        const int sub = lane & (TPC - 1);
        const int cpi = G >> tpc_log2;  // channels per iteration of the slot
        for (int d0 = 0; d0 < s.D; d0 += cpi) {
          const int d = d0 + (lane >> tpc_log2);
          float ag = 0.0f, ab = 0.0f;
          if (d < s.D) {
            const int q0 = STRADDLE ? (d * s.HxW + E - 1) / E : d * S;
            const int q1 = STRADDLE ? ((d + 1) * s.HxW + E - 1) / E : (d + 1) * S;
            for (int q = q0 + sub; q < q1; q += TPC) {
              ag += st[2 * q];
              ab += st[2 * q + 1];
            }
            if constexpr (STRADDLE) {
              // the channel starts inside a pack: that pack's share of it
              if (sub == 0 && (d * s.HxW) % E != 0) {
                ag += sn[2 * d];
                ab += sn[2 * d + 1];
              }
            }
          }
          for (int off = TPC >> 1; off > 0; off >>= 1) {
            ag += __shfl_xor(ag, off, 64);
            ab += __shfl_xor(ab, off, 64);
          }
          if (ok && d < s.D && sub == 0) {
            const int64_t n = row / s.groups;
            const int64_t o = n * ((int64_t)s.groups * s.D) + (int64_t)g * s.D + d;
            part_dg[o] = ag;
            if (part_db) part_db[o] = ab;
          }
        }
        __syncthreads();  // the staging area is reused by the next row
      }
    }
  }
}

// ---------------------------------------------------------------------------
// The same backward for the rows gn_fwd_exact_kernel serves (L == G * V * E, one
// row a workgroup, channels of whole runs of 64 packs, dx written): scalar row
// pointers, statistics and weights, no conditional access.  The 64 packs of a
// wavefront lie in one channel, so the sums over a pack are reduced over the
// wavefront in registers and one lane parks them in LDS ahead of the barrier the
// row's reduction has anyway; after it every wavefront adds the runs of each
// channel in a fixed order and all of them write the row's D channel sums, the
// same values to the same addresses: a store by the first wavefront only would be
// a conditional store, and the compiler then lets the next row's loads wait for
// it.  dx is that of gn_bwd_resident_kernel for the same layout, bit for bit; the
// channel sums differ from it in the last bits (another order of the same terms).
// Measured on one MI355X, bf16 [64, 320, 64, 64] with 32 groups on 512 lanes x 10
// packs, two workgroups a compute unit: 92.7 -> 87.0 us (before the column pass).
template <class T, class WT, int G, int V, bool COLS>
__global__ void __launch_bounds__(G)
gn_bwd_exact_kernel(const T* __restrict__ dy, const T* __restrict__ x,
                    const WT* __restrict__ mean, const WT* __restrict__ rstd,
                    const WT* __restrict__ gamma, T* __restrict__ dx,
                    float* __restrict__ part_dg, float* __restrict__ part_db, int64_t rows,
                    GroupShape s) {
  constexpr int E = elems_per_pack<T>::value;
  constexpr int NW = G / 64;
  constexpr int UNITS = V * NW;  // runs of 64 packs in a row
  static_assert(sizeof(T) == 2 && G % 64 == 0, "16-bit rows on whole wavefronts");
  __shared__ float red[reduce_lds_floats<G, G, 2>::value];
  __shared__ float stage[COLS ? 2 * UNITS * 2 : 1];  // [phase][run][dg, db]
  int phase = 0;
  const float fL = (float)s.L;
  const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
  const int lane = (int)(threadIdx.x & 63);
  const unsigned S = (unsigned)(s.HxW / E);  // packs per channel
  const int U = (int)(S / 64u);              // runs per channel
  int chl[V];
#pragma unroll
  for (int c = 0; c < V; ++c) chl[c] = (int)((unsigned)(c * G + wave * 64) / S);
  // the channel whose sums this lane writes; lanes beyond the row's channels repeat one
  const int dch = lane % s.D;
  const uint32_t loff = (uint32_t)(threadIdx.x * E * (int)sizeof(T));
  auto at = [](const T* p, uint32_t off) {
    return reinterpret_cast<const T*>(reinterpret_cast<const char*>(p) + off);
  };
  const bool has_g = gamma != nullptr;
  const WT* gsrc = has_g ? gamma : reinterpret_cast<const WT*>(x);
  for (int64_t row = blockIdx.x; row < rows; row += gridDim.x) {
    const uint32_t n = (uint32_t)row / (uint32_t)s.groups;
    const int ch0 = (int)((uint32_t)row - n * (uint32_t)s.groups) * s.D;
    const UniformElem<WT> wmu = UniformElem<WT>::load(mean, row);
    const UniformElem<WT> wrs = UniformElem<WT>::load(rstd, row);
    const T* xr = x + row * (int64_t)s.L;
    const T* gr = dy + row * (int64_t)s.L;
    UniformElem<WT> wg[V];
    Pack<T, E> xp[V], dp[V];
#pragma unroll
    for (int c = 0; c < V; ++c) {
      wg[c] = UniformElem<WT>::load(gsrc, ch0 + chl[c]);
      xp[c] = Pack<T, E>::load_stream(at(xr + c * G * E, loff));
      dp[c] = Pack<T, E>::load_stream(at(gr + c * G * E, loff));
    }
    const float mu = wmu.value(), rs = wrs.value();
    float ga[V];
    float acc[2] = {0.0f, 0.0f};
    float* st = stage + phase * (2 * UNITS);
#pragma unroll
    for (int c = 0; c < V; ++c) {
      ga[c] = has_g ? wg[c].value() : 1.0f;
      float pdg = 0.0f, pdb = 0.0f;
#pragma unroll
      for (int i = 0; i < E; ++i) {
        const float gy = dp[c].get(i);
        pdb += gy;
        pdg = fmaf(gy, xp[c].get(i) - mu, pdg);
      }
      acc[0] = fmaf(pdb, ga[c], acc[0]);
      acc[1] = fmaf(pdg * rs, ga[c], acc[1]);
      if constexpr (COLS) {
        const float wdg = wave_group_allreduce<64, SumOp>(pdg * rs);
        const float wdb = wave_group_allreduce<64, SumOp>(pdb);
        if (lane == 0) {
          st[2 * (c * NW + wave)] = wdg;
          st[2 * (c * NW + wave) + 1] = wdb;
        }
      }
    }
    group_allreduce<G, G, 2, SumOp>(acc, red, phase);  // (flips phase)
    if constexpr (COLS) {
      float ag = 0.0f, ab = 0.0f;
      for (int u = 0; u < U; ++u) {
        ag += st[2 * (dch * U + u)];
        ab += st[2 * (dch * U + u) + 1];
      }
      const int64_t o = (int64_t)n * ((int64_t)s.groups * s.D) + ch0 + dch;
      part_dg[o] = ag;
      part_db[o] = ab;
    }
    T* dr = dx + row * (int64_t)s.L;
    const float s1 = acc[0], s2 = acc[1];
    const float term1 = rs / fL;
    const float ra = rs * (s2 * term1);
    const float cc = mu * ra - s1 * term1;
#pragma unroll
    for (int c = 0; c < V; ++c) {
      keep_packed(xp[c]);
      keep_packed(dp[c]);
      const float gq = ga[c] * rs;
      Pack<T, E> o;
#pragma unroll
      for (int i = 0; i < E; ++i) o.set(i, fmaf(xp[c].get(i), -ra, fmaf(dp[c].get(i), gq, cc)));
      o.store_stream(const_cast<T*>(at(dr + c * G * E, loff)));
    }
  }
}

// Backward dX for rows too long for the registers, from the per-(n, channel)
// sums that gn_channel_sums_kernel left in part_dg / part_db: every workgroup
// takes one chunk of BLOCK * CHUNK_PACKS packs of one row, rebuilds the row's
// s1 = sum_c gamma*db and s2 = sum_c gamma*dg from the D channel sums (the
// reference's ComputeBackwardFusedParamsFunctor, GroupNormKernels.cpp:
// 1088-1165) and then works element by element, so a few very long rows still
// spread over the whole machine.
constexpr int kGnChunkPacks = 8;

template <class T, class WT, int BLOCK>
__global__ void __launch_bounds__(BLOCK)
gn_bwd_dx_from_sums_kernel(const T* __restrict__ dy, const T* __restrict__ x,
                           const WT* __restrict__ mean, const WT* __restrict__ rstd,
                           const WT* __restrict__ gamma, const float* __restrict__ part_dg,
                           const float* __restrict__ part_db, T* __restrict__ dx, int64_t rows,
                           GroupShape s, int chunks_per_row) {
  constexpr int E = elems_per_pack<T>::value;
  __shared__ float red[reduce_lds_floats<BLOCK, BLOCK, 2>::value];
  int phase = 0;
  const float fL = (float)s.L;
  const int64_t ntiles = rows * chunks_per_row;
  const bool uniform = (s.HxW % E) == 0;
  for (int64_t t = blockIdx.x; t < ntiles; t += gridDim.x) {
    const int64_t row = t / chunks_per_row;
    const int chunk = (int)(t - row * chunks_per_row);
    const int g = (int)((uint32_t)row % (uint32_t)s.groups);
    const int64_t n = row / s.groups;
    const float mu = (float)mean[row], rs = (float)rstd[row];
    const int64_t c0 = n * ((int64_t)s.groups * s.D) + (int64_t)g * s.D;
    float acc[2] = {0.0f, 0.0f};
    for (int d = threadIdx.x; d < s.D; d += BLOCK) {
      const float ga = gn_weight(gamma, g * s.D + d, 1.0f);
      acc[0] = fmaf(part_db[c0 + d], ga, acc[0]);
      acc[1] = fmaf(part_dg[c0 + d], ga, acc[1]);
    }
    group_allreduce<BLOCK, BLOCK, 2, SumOp>(acc, red, phase);
    const float s1 = acc[0], s2 = acc[1], term1 = rs / fL;
    const T* xr = x + row * (int64_t)s.L;
    const T* gr = dy + row * (int64_t)s.L;
    T* dr = dx + row * (int64_t)s.L;
    // A chunk that lies wholly inside a row whose channels are whole packs: straight-line
    // code, all 2 * kGnChunkPacks loads of a lane requested before the first is used and
    // one weight a pack (the general loop below tests every pack against the row end and
    // the weight pointer, and each such branch waits for what is outstanding).
    const int64_t pk_first = (int64_t)chunk * kGnChunkPacks * BLOCK;
    if (uniform && gamma != nullptr && (pk_first + (int64_t)kGnChunkPacks * BLOCK) * E <= s.L) {
      const uint32_t pk0 = (uint32_t)pk_first + threadIdx.x;
      const uint32_t S = (uint32_t)(s.HxW / E);  // packs a channel
      Pack<T, E> px[kGnChunkPacks], pd[kGnChunkPacks];
      WT gw[kGnChunkPacks];
#pragma unroll
      for (int k = 0; k < kGnChunkPacks; ++k) {
        const uint32_t pk = pk0 + (uint32_t)(k * BLOCK);
        px[k] = Pack<T, E>::load_stream(xr + (int64_t)pk * E);
        pd[k] = Pack<T, E>::load_stream(gr + (int64_t)pk * E);
        gw[k] = gamma[g * s.D + (int)(pk / S)];
      }
#pragma unroll
      for (int k = 0; k < kGnChunkPacks; ++k) {
        const uint32_t pk = pk0 + (uint32_t)(k * BLOCK);
        const float ga = (float)gw[k];
        Pack<T, E> o;
#pragma unroll
        for (int i = 0; i < E; ++i) {
          float f = fL * (pd[k].get(i) * ga);
          f -= ((px[k].get(i) - mu) * rs) * s2;
          f -= s1;
          o.set(i, f * term1);
        }
        o.store_stream(dr + (int64_t)pk * E);
      }
      continue;
    }
#pragma unroll
    for (int k = 0; k < kGnChunkPacks; ++k) {
      const int64_t pk = ((int64_t)chunk * kGnChunkPacks + k) * BLOCK + threadIdx.x;
      const int64_t e64 = pk * E;
      const int e0 = e64 < s.L ? (int)e64 : s.L;
      const Pack<T, E> px = load_row_pack<T, E, true>(xr, e0, s.L, true, 0.0f);
      const Pack<T, E> pd = load_row_pack<T, E, true>(gr, e0, s.L, true, 0.0f);
      const float gu = gn_weight(gamma, gn_channel(s, g, e0), 1.0f);
      Pack<T, E> o;
#pragma unroll
      for (int i = 0; i < E; ++i) {
        const float ga = uniform ? gu : gn_weight(gamma, gn_channel(s, g, e0 + i), 1.0f);
        float f = fL * (pd.get(i) * ga);
        f -= ((px.get(i) - mu) * rs) * s2;
        f -= s1;
        o.set(i, f * term1);
      }
      store_row_pack<T, E, true>(dr, e0, s.L, true, o);
    }
  }
}

// Per-(n, channel) sums of dy*xhat and dy for the cases the fused path does not
// cover.  LANES lanes walk one channel row of HxW contiguous elements: a power
// of two up to 64 (a wavefront then holds 64 / LANES rows, reduced with
// shuffles), or the whole workgroup for long channel rows (reduced through LDS).
template <class T, class WT, int BLOCK>
__global__ void __launch_bounds__(BLOCK)
gn_channel_sums_kernel(const T* __restrict__ dy, const T* __restrict__ x,
                       const WT* __restrict__ mean, const WT* __restrict__ rstd,
                       float* __restrict__ part_dg, float* __restrict__ part_db, int64_t nc_rows,
                       GroupShape s, int lanes_log2) {
  constexpr int E = elems_per_pack<T>::value;
  __shared__ float red[reduce_lds_floats<BLOCK, BLOCK, 2>::value];
  int phase = 0;
  const int LANES = 1 << lanes_log2;
  const bool whole_block = LANES == BLOCK;  // uniform
  const int sub = threadIdx.x & (LANES - 1);
  const int rpb = BLOCK >> lanes_log2;  // channel rows per workgroup iteration
  const int npacks = (s.HxW + E - 1) / E;
  const int C = s.groups * s.D;
  const int64_t nrb = (nc_rows + rpb - 1) / rpb;
  for (int64_t rb = blockIdx.x; rb < nrb; rb += gridDim.x) {
    const int64_t r = rb * rpb + (threadIdx.x >> lanes_log2);  // n * C + c
    const bool ok = r < nc_rows;
    const int64_t rc = ok ? r : 0;
    const int64_t n = rc / C;
    const int c = (int)(rc - n * C);
    const int64_t srow = n * s.groups + c / s.D;
    const float mu = (float)mean[srow], rs = (float)rstd[srow];
    const T* xr = x + rc * (int64_t)s.HxW;
    const T* gr = dy + rc * (int64_t)s.HxW;
    float acc[2] = {0.0f, 0.0f};
    int pk = sub;
    if ((s.HxW % E) == 0) {
      // channels of whole packs: four pack pairs a lane in flight, nothing conditional
      // (a row slot past the last row reads row 0 and stores nothing)
      constexpr int U = 4;
      for (; pk + (U - 1) * LANES < npacks; pk += U * LANES) {
        Pack<T, E> px[U], pd[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
          px[u] = Pack<T, E>::load_stream(xr + (int64_t)(pk + u * LANES) * E);
          pd[u] = Pack<T, E>::load_stream(gr + (int64_t)(pk + u * LANES) * E);
        }
#pragma unroll
        for (int u = 0; u < U; ++u)
#pragma unroll
          for (int i = 0; i < E; ++i) {
            const float gy = pd[u].get(i);
            acc[1] += gy;
            acc[0] = fmaf(gy, px[u].get(i) - mu, acc[0]);
          }
      }
    }
    for (; pk < npacks; pk += LANES) {
      const Pack<T, E> px = load_row_pack<T, E, true>(xr, pk * E, s.HxW, ok, 0.0f);
      const Pack<T, E> pd = load_row_pack<T, E, true>(gr, pk * E, s.HxW, ok, 0.0f);
      const int nvalid = s.HxW - pk * E;
#pragma unroll
      for (int i = 0; i < E; ++i) {
        const float gy = pd.get(i);
        acc[1] += gy;
        acc[0] = fmaf(gy, i < nvalid ? px.get(i) - mu : 0.0f, acc[0]);
      }
    }
    if (whole_block) {
      group_allreduce<BLOCK, BLOCK, 2, SumOp>(acc, red, phase);
    } else {
      for (int off = LANES >> 1; off > 0; off >>= 1) {
        acc[0] += __shfl_xor(acc[0], off, 64);
        acc[1] += __shfl_xor(acc[1], off, 64);
      }
    }
    if (ok && sub == 0) {
      part_dg[r] = acc[0] * rs;
      if (part_db) part_db[r] = acc[1];
    }
  }
}

// ---------------------------------------------------------------------------
// Backward of slabs beyond one workgroup's registers whose channels are whole packs, dY and
// X read once: a team of workgroups holds a (sample, group) slab, `wpc` workgroups a channel,
// V packs of dY and of X a lane.  A workgroup publishes its piece's sums of dy * (x - mean)
// * rstd and of dy (team_publish_and_gather); every workgroup adds the team's numbers channel
// by channel in a fixed order, forms s1 = sum_c gamma_c * db_c and s2 = sum_c gamma_c * dg_c
// (the reference's ComputeBackwardFusedParamsFunctor, GroupNormKernels.cpp:1088-1165) and
// writes dX for what it holds; the first workgroup of a channel leaves the channel's sums in
// the [N, C] partial buffers (the second stage adds them over the samples).  A workgroup
// whose wait runs out takes the slab's sums itself in a pass over the whole slab (dX must
// not overlap dY or X) and loads its packs again.
template <class T, class WT, int V>
__global__ void __launch_bounds__(kTeamBlock, kTeamPerCu * kTeamBlock / 256)
gn_bwd_team_kernel(const T* __restrict__ dy, const T* __restrict__ x,
                   const WT* __restrict__ mean, const WT* __restrict__ rstd,
                   const WT* __restrict__ gamma, T* __restrict__ dx,
                   float* __restrict__ part_dg, float* __restrict__ part_db, int64_t rows,
                   GroupShape s, int team, int wpc, TeamSlot* slot, unsigned int call_id,
                   unsigned long long wait_ticks) {
  constexpr int E = elems_per_pack<T>::value;
  constexpr int BLOCK = kTeamBlock;
  __shared__ float red[reduce_lds_floats<BLOCK, BLOCK, 4>::value];
  __shared__ double tpart[kTeamMaxWorkgroups][2];
  __shared__ float stat[4];  // s1, s2, -, whether the team failed
  int phase = 0;
  const int tm = (int)blockIdx.x / team;
  const int c = (int)blockIdx.x - tm * team;
  const int teams = (int)gridDim.x / team;
  const int ch = c / wpc;             // the channel of the group this workgroup works on
  const int piece = c - ch * wpc;     // and its piece of the channel
  const int cp = s.HxW / E;           // packs a channel
  const int pk0 = piece * (V * BLOCK) + (int)threadIdx.x;
  const float fL = (float)s.L;
  const uint32_t loff = (uint32_t)(pk0 < cp ? pk0 : 0) * 16u;
  // (a pointer into global memory, as in the other team kernels)
  auto at = [](auto* p, uint32_t off) {
    using Elem = std::remove_pointer_t<decltype(p)>;
    typedef __attribute__((address_space(1))) Elem* GlobalPtr;
    return (Elem*)reinterpret_cast<GlobalPtr>(reinterpret_cast<uintptr_t>(p) + off);
  };
  unsigned int round = 0;
  for (int64_t row = tm; row < rows; row += teams, ++round) {
    TeamEntry* entries = slot->entry[round & 1u];
    if (threadIdx.x == 0) team_store(&entries[blockIdx.x].tag, 0ull);
    const int g = (int)((uint32_t)row % (uint32_t)s.groups);
    const int64_t n = row / s.groups;
    const float mu = (float)mean[row], rs = (float)rstd[row];
    const int64_t base = row * (int64_t)s.L + (int64_t)ch * s.HxW;
    const T* gb = dy + base;
    const T* xb = x + base;
    Pack<T, E> dp[V], xp[V];
    auto load_chunk = [&]() {
#pragma unroll
      for (int k = 0; k < V; ++k) {
        dp[k] = Pack<T, E>::zero();
        xp[k] = Pack<T, E>::zero();
        if (pk0 + k * BLOCK < cp) {
          dp[k] = Pack<T, E>::load_stream(at(gb + k * BLOCK * E, loff));
          xp[k] = Pack<T, E>::load_stream(at(xb + k * BLOCK * E, loff));
        }
      }
    };
    load_chunk();
    float acc[2] = {0.0f, 0.0f};
#pragma unroll
    for (int k = 0; k < V; ++k) {
      if (pk0 + k * BLOCK < cp) {
#pragma unroll
        for (int i = 0; i < E; ++i) {
          const float gy = dp[k].get(i);
          acc[1] += gy;
          acc[0] = fmaf(gy, xp[k].get(i) - mu, acc[0]);
        }
      }
      keep_packed(dp[k]);
      keep_packed(xp[k]);
      __builtin_amdgcn_sched_barrier(0);  // (one pack widened at a time: registers)
    }
    group_allreduce<BLOCK, BLOCK, 2, SumOp>(acc, red, phase);
    if (threadIdx.x < 64) {  // the first wavefront publishes, waits and adds up
      const int lane = (int)threadIdx.x;
      const bool complete =
          team_publish_and_gather(slot, entries, tm, team, call_id, round, wait_ticks,
                                  (double)(acc[0] * rs), (double)acc[1], tpart);
      // (the lanes of a wavefront see one another's LDS stores in program order)
      if (complete) {
        float s1 = 0.0f, s2 = 0.0f;
        for (int d = lane; d < s.D; d += 64) {
          float dg = 0.0f, db = 0.0f;
          for (int q = 0; q < wpc; ++q) {
            dg += (float)tpart[d * wpc + q][0];
            db += (float)tpart[d * wpc + q][1];
          }
          const float ga = gn_weight(gamma, g * s.D + d, 1.0f);
          s1 = fmaf(db, ga, s1);
          s2 = fmaf(dg, ga, s2);
          if (d == ch && piece == 0 && part_dg != nullptr) {
            const int64_t o = n * ((int64_t)s.groups * s.D) + (int64_t)g * s.D + d;
            part_dg[o] = dg;
            if (part_db != nullptr) part_db[o] = db;
          }
        }
        s1 = wave_group_allreduce<64, SumOp>(s1);
        s2 = wave_group_allreduce<64, SumOp>(s2);
        if (lane == 0) {
          stat[0] = s1;
          stat[1] = s2;
          stat[3] = 0.0f;
        }
      } else if (lane == 0) {
        stat[3] = 1.0f;
      }
    }
    __syncthreads();
    if (stat[3] != 0.0f) {  // (uniform over the workgroup)
      // The team did not come together: the slab's sums in a pass over the whole slab --
      // s1, s2 and, for the partial buffers, this workgroup's own channel --, then the
      // packs again.
      const T* gr = dy + row * (int64_t)s.L;
      const T* xr = x + row * (int64_t)s.L;
      float w[4] = {0.0f, 0.0f, 0.0f, 0.0f};  // s1, s2 / rstd, own channel's dg / rstd and db
      for (int pk = (int)threadIdx.x; pk < s.D * cp; pk += BLOCK) {
        const int d = pk / cp;
        const Pack<T, E> pd = Pack<T, E>::load(gr + (int64_t)pk * E);
        const Pack<T, E> px = Pack<T, E>::load(xr + (int64_t)pk * E);
        const float ga = gn_weight(gamma, g * s.D + d, 1.0f);
        float a = 0.0f, b = 0.0f;
#pragma unroll
        for (int i = 0; i < E; ++i) {
          const float gy = pd.get(i);
          b += gy;
          a = fmaf(gy, px.get(i) - mu, a);
        }
        w[0] = fmaf(b, ga, w[0]);
        w[1] = fmaf(a, ga, w[1]);
        if (d == ch) {
          w[2] += a;
          w[3] += b;
        }
      }
      group_allreduce<BLOCK, BLOCK, 4, SumOp>(w, red, phase);
      if (threadIdx.x == 0) {
        stat[0] = w[0];
        stat[1] = w[1] * rs;
        if (piece == 0 && part_dg != nullptr) {
          const int64_t o = n * ((int64_t)s.groups * s.D) + (int64_t)g * s.D + ch;
          part_dg[o] = w[2] * rs;
          if (part_db != nullptr) part_db[o] = w[3];
        }
      }
      __syncthreads();
      load_chunk();
    }
    const float s1 = stat[0], s2 = stat[1], term1 = rs / fL;
    const float ga = gn_weight(gamma, g * s.D + ch, 1.0f);
    T* ob = dx + base;
#pragma unroll
    for (int k = 0; k < V; ++k) {
      if (pk0 + k * BLOCK < cp) {
        Pack<T, E> o;
#pragma unroll
        for (int i = 0; i < E; ++i) {
          float f = fL * (dp[k].get(i) * ga);
          f -= ((xp[k].get(i) - mu) * rs) * s2;
          f -= s1;
          o.set(i, f * term1);
        }
        o.store_stream(at(ob + k * BLOCK * E, loff));
      }
      // (pack k + 1 is widened after pack k has been stored, not before: registers)
      __builtin_amdgcn_sched_barrier(0);
    }
    // stat[] is rewritten for the next slab only after every thread has passed the
    // barrier of the next block reduction, i.e. after it has read this slab's values
  }
}

}  // namespace rownorm
