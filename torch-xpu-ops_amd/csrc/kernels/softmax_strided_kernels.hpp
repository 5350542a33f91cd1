// softmax / log_softmax over a dimension that is NOT innermost, on a dense
// tensor viewed as [outer, D, inner] (inner > 1 contiguous elements).
//
// Every one of the `inner` columns of an [D, inner] slab is its own softmax
// problem whose D elements lie `inner` apart in memory.  A group of TX * TY
// threads takes a tile of TX consecutive 16-byte packs of the inner dimension
// and all D rows: thread (ty, tx) holds the packs of rows ty, ty + TY, ... of
// pack column tx in registers (V packs), so each lane keeps E independent
// running maxima and sums, one per element of its pack.  The TX lanes of a row
// read one contiguous TX * 16 byte segment.  The reduction over D runs across
// the TY threads that share tx: butterfly shuffles inside a wavefront and, only
// when a group is wider than a wavefront, one LDS exchange among its
// wavefronts.  A workgroup holds BLOCK / (TX * TY) such groups, each on its own
// tile.  X is read once and Y written once.
//
// Stands in for SpatialSoftmaxForwardKernelFunctor (src/ATen/native/xpu/sycl/
// SoftMaxKernels.cpp:725-950) and SpatialSoftmaxBackwardKernelFunctor
// (:1387-1564), which walk the D rows three times (max, sum, output) from
// global memory; the dispatch they sit behind is :1721-1736.  D too large for
// the registers takes the multi-pass kernels at the end of this file, which do
// the same walk.
#pragma once
#include "device/pack.hpp"
#include "device/reduce.hpp"
#include "launch.hpp"
#include "softmax_kernels.hpp"

namespace rownorm {

// LDS floats for column_allreduce in a BLOCK-thread workgroup of E-element packs.
template <int BLOCK, int E>
struct column_lds_floats {
  static constexpr int value = 2 * (BLOCK / 64) * 64 * E;
};

// Thread layout of one workgroup: threadIdx.x = (group * TY + ty) * TX + tx.
struct StridedLayout {
  int tx_log2, ty_log2;
};

// All-reduce of the E values of every lane over the TY threads of its group
// that share tx (TX, TY powers of two, TX <= 64, TX * TY <= BLOCK).  Fixed
// order; every thread of the workgroup must call it (it holds a barrier when
// a group spans several wavefronts).
template <int BLOCK, int E, class Op>
__device__ __forceinline__ void column_allreduce(float (&v)[E], StridedLayout lay, float* lds,
                                                 int& phase) {
  const int TX = 1 << lay.tx_log2;
  const int GT = TX << lay.ty_log2;  // threads per group
  const int span = GT < 64 ? GT : 64;
  for (int off = TX; off < span; off <<= 1) {
#pragma unroll
    for (int i = 0; i < E; ++i) v[i] = Op::apply(v[i], __shfl_xor(v[i], off, 64));
  }
  constexpr int NW = BLOCK / 64;
  if (GT > 64) {  // uniform over the workgroup
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int wpg = GT >> 6;  // wavefronts per group
    float* buf = lds + phase * (NW * 64 * E);
    if (lane < TX) {
#pragma unroll
      for (int i = 0; i < E; ++i) buf[(wave * 64 + lane) * E + i] = v[i];
    }
    __syncthreads();
    const int tx = lane & (TX - 1);
    const int w0 = wave & ~(wpg - 1);
#pragma unroll
    for (int i = 0; i < E; ++i) {
      float acc = buf[(w0 * 64 + tx) * E + i];
      for (int w = 1; w < wpg; ++w) acc = Op::apply(acc, buf[((w0 + w) * 64 + tx) * E + i]);
      v[i] = acc;
    }
    phase ^= 1;
  }
}

// The tile a thread works on in one iteration of its workgroup.
struct StridedTile {
  int64_t slab;  // element offset of the [D, inner] slab
  int e0;        // first inner element of this lane's pack (== inner when out of range)
  int ty, TY;
  bool valid;    // false: the group has run out of tiles; nothing is loaded or stored
};

template <int BLOCK, int E>
__device__ __forceinline__ StridedTile strided_tile(int64_t t0, int64_t ntiles, int64_t xtiles,
                                                    int D, int inner, StridedLayout lay) {
  const int TX = 1 << lay.tx_log2;
  const int tx = threadIdx.x & (TX - 1);
  const int rest = threadIdx.x >> lay.tx_log2;
  StridedTile r;
  r.TY = 1 << lay.ty_log2;
  r.ty = rest & (r.TY - 1);
  const int64_t t = t0 + (rest >> lay.ty_log2);
  r.valid = t < ntiles;
  const int64_t tc = r.valid ? t : 0;
  const int64_t o = tc / xtiles;
  const int64_t xt = tc - o * xtiles;
  r.slab = o * (int64_t)D * (int64_t)inner;
  const int64_t e = (xt * TX + tx) * (int64_t)E;
  r.e0 = e < inner ? (int)e : inner;
  return r;
}

// Tiles a workgroup takes per iteration, and the tile count of the problem.
template <int BLOCK>
__device__ __forceinline__ int groups_per_block(StridedLayout lay) {
  return BLOCK >> (lay.tx_log2 + lay.ty_log2);
}

template <class TI, class TO, int V, int BLOCK, bool FAST>
__global__ void __launch_bounds__(BLOCK)
softmax_strided_fwd_kernel(const TI* __restrict__ x, TO* __restrict__ y, int64_t outer, int D,
                           int inner, StridedLayout lay, int flags) {
  constexpr int E = elems_per_pack<TI>::value;
  constexpr bool PRECISE = sizeof(TO) == 4;
  __shared__ float red[column_lds_floats<BLOCK, E>::value];
  int phase = 0;
  const bool is_log = (flags & kSoftmaxLog) != 0;
  const bool is_safe = (flags & kSoftmaxSafe) != 0;
  const int64_t xtiles = (((inner + E - 1) / E) + (1 << lay.tx_log2) - 1) >> lay.tx_log2;
  const int64_t ntiles = outer * xtiles;
  const int NG = groups_per_block<BLOCK>(lay);
  for (int64_t t0 = (int64_t)blockIdx.x * NG; t0 < ntiles; t0 += (int64_t)gridDim.x * NG) {
    const StridedTile tile = strided_tile<BLOCK, E>(t0, ntiles, xtiles, D, inner, lay);
    const int ty = tile.ty, TY = tile.TY;
    // the V packs stay in storage format; each pass widens them again (softmax
    // then evaluates exp twice per element, which measured faster than holding
    // V * E fp32 values a lane)
    Pack<TI, E> xp[V];
#pragma unroll
    for (int k = 0; k < V; ++k) {
      const int d = ty + k * TY;
      const bool ok = tile.valid && d < D;
      const TI* row = x + tile.slab + (int64_t)(ok ? d : 0) * inner;
      xp[k] = row_load<TI, E, true, FAST>(row, tile.e0, inner, ok, -INFINITY);
    }
    float mx[E], sum[E];
#pragma unroll
    for (int i = 0; i < E; ++i) {
      mx[i] = -INFINITY;
#pragma unroll
      for (int k = 0; k < V; ++k) mx[i] = fmaxf(mx[i], xp[k].get(i));
    }
    column_allreduce<BLOCK, E, MaxOp>(mx, lay, red, phase);
#pragma unroll
    for (int i = 0; i < E; ++i) sum[i] = 0.0f;
#pragma unroll
    for (int k = 0; k < V; ++k) {
      keep_packed(xp[k]);
#pragma unroll
      for (int i = 0; i < E; ++i) sum[i] += row_exp<PRECISE>(xp[k].get(i) - mx[i]);
    }
    column_allreduce<BLOCK, E, SumOp>(sum, lay, red, phase);
    // one scalar branch per run-time variant (see ROWNORM_UNIFORM_ARM)
    float kf[E];
    if (is_log) {
      ROWNORM_UNIFORM_ARM("log_softmax over a strided dimension");
#pragma unroll
      for (int i = 0; i < E; ++i) kf[i] = logf(sum[i]);
#pragma unroll
      for (int k = 0; k < V; ++k) {
        keep_packed(xp[k]);
        const int d = ty + k * TY;
        const bool ok = tile.valid && d < D;
        Pack<TO, E> o;
#pragma unroll
        for (int i = 0; i < E; ++i) o.set(i, (xp[k].get(i) - mx[i]) - kf[i]);
        TO* row = y + tile.slab + (int64_t)(ok ? d : 0) * inner;
        row_store<TO, E, true, FAST>(row, tile.e0, inner, ok, o);
      }
    } else if (is_safe) {
      ROWNORM_UNIFORM_ARM("safe softmax over a strided dimension");
      bool zero[E];
#pragma unroll
      for (int i = 0; i < E; ++i) {
        kf[i] = 1.0f / sum[i];
        zero[i] = mx[i] == -INFINITY;
      }
#pragma unroll
      for (int k = 0; k < V; ++k) {
        keep_packed(xp[k]);
        const int d = ty + k * TY;
        const bool ok = tile.valid && d < D;
        Pack<TO, E> o;
#pragma unroll
        for (int i = 0; i < E; ++i)
          o.set(i, zero[i] ? 0.0f : row_exp<PRECISE>(xp[k].get(i) - mx[i]) * kf[i]);
        TO* row = y + tile.slab + (int64_t)(ok ? d : 0) * inner;
        row_store<TO, E, true, FAST>(row, tile.e0, inner, ok, o);
      }
    } else {
      ROWNORM_UNIFORM_ARM("softmax over a strided dimension");
#pragma unroll
      for (int i = 0; i < E; ++i) kf[i] = 1.0f / sum[i];
#pragma unroll
      for (int k = 0; k < V; ++k) {
        keep_packed(xp[k]);
        const int d = ty + k * TY;
        const bool ok = tile.valid && d < D;
        Pack<TO, E> o;
#pragma unroll
        for (int i = 0; i < E; ++i) o.set(i, row_exp<PRECISE>(xp[k].get(i) - mx[i]) * kf[i]);
        TO* row = y + tile.slab + (int64_t)(ok ? d : 0) * inner;
        row_store<TO, E, true, FAST>(row, tile.e0, inner, ok, o);
      }
    }
  }
}

// TG: dtype of grad and of the saved output y; TO: dtype of the input gradient.
template <class TG, class TO, int V, int BLOCK, bool FAST>
__global__ void __launch_bounds__(BLOCK)
softmax_strided_bwd_kernel(const TG* __restrict__ grad, const TG* __restrict__ y,
                           TO* __restrict__ gi, int64_t outer, int D, int inner, StridedLayout lay,
                           int flags) {
  constexpr int E = elems_per_pack<TG>::value;
  constexpr bool PRECISE = sizeof(TO) == 4 && sizeof(TG) == 4;
  __shared__ float red[column_lds_floats<BLOCK, E>::value];
  int phase = 0;
  const bool is_log = (flags & kSoftmaxLog) != 0;
  const int64_t xtiles = (((inner + E - 1) / E) + (1 << lay.tx_log2) - 1) >> lay.tx_log2;
  const int64_t ntiles = outer * xtiles;
  const int NG = groups_per_block<BLOCK>(lay);
  for (int64_t t0 = (int64_t)blockIdx.x * NG; t0 < ntiles; t0 += (int64_t)gridDim.x * NG) {
    const StridedTile tile = strided_tile<BLOCK, E>(t0, ntiles, xtiles, D, inner, lay);
    const int ty = tile.ty, TY = tile.TY;
    Pack<TG, E> pg[V], py[V];
#pragma unroll
    for (int k = 0; k < V; ++k) {
      const int d = ty + k * TY;
      const bool ok = tile.valid && d < D;
      const int64_t off = tile.slab + (int64_t)(ok ? d : 0) * inner;
      pg[k] = row_load<TG, E, true, FAST>(grad + off, tile.e0, inner, ok, 0.0f);
      py[k] = row_load<TG, E, true, FAST>(y + off, tile.e0, inner, ok, 0.0f);
    }
    float sum[E];
#pragma unroll
    for (int i = 0; i < E; ++i) sum[i] = 0.0f;
    if (is_log) {
      ROWNORM_UNIFORM_ARM("log_softmax backward over a strided dimension: sum of grad");
#pragma unroll
      for (int i = 0; i < E; ++i)
#pragma unroll
        for (int k = 0; k < V; ++k) sum[i] += pg[k].get(i);
    } else {
      ROWNORM_UNIFORM_ARM("softmax backward over a strided dimension: sum of y * grad");
#pragma unroll
      for (int i = 0; i < E; ++i)
#pragma unroll
        for (int k = 0; k < V; ++k) sum[i] = fmaf(py[k].get(i), pg[k].get(i), sum[i]);
    }
    column_allreduce<BLOCK, E, SumOp>(sum, lay, red, phase);
    if (is_log) {
      ROWNORM_UNIFORM_ARM("log_softmax backward over a strided dimension");
#pragma unroll
      for (int k = 0; k < V; ++k) {
        const int d = ty + k * TY;
        const bool ok = tile.valid && d < D;
        Pack<TO, E> o;
#pragma unroll
        for (int i = 0; i < E; ++i)
          o.set(i, pg[k].get(i) - row_exp<PRECISE>(py[k].get(i)) * sum[i]);
        TO* row = gi + tile.slab + (int64_t)(ok ? d : 0) * inner;
        row_store<TO, E, true, FAST>(row, tile.e0, inner, ok, o);
      }
    } else {
      ROWNORM_UNIFORM_ARM("softmax backward over a strided dimension");
#pragma unroll
      for (int k = 0; k < V; ++k) {
        const int d = ty + k * TY;
        const bool ok = tile.valid && d < D;
        Pack<TO, E> o;
#pragma unroll
        for (int i = 0; i < E; ++i) o.set(i, py[k].get(i) * (pg[k].get(i) - sum[i]));
        TO* row = gi + tile.slab + (int64_t)(ok ? d : 0) * inner;
        row_store<TO, E, true, FAST>(row, tile.e0, inner, ok, o);
      }
    }
  }
}

// D beyond the register budget: same tiling, the D rows are walked three times
// (forward) or twice (backward) from memory.
template <class TI, class TO, int BLOCK>
__global__ void __launch_bounds__(BLOCK)
softmax_strided_fwd_stream_kernel(const TI* __restrict__ x, TO* __restrict__ y, int64_t outer,
                                  int D, int inner, StridedLayout lay, int flags) {
  constexpr int E = elems_per_pack<TI>::value;
  constexpr bool PRECISE = sizeof(TO) == 4;
  __shared__ float red[column_lds_floats<BLOCK, E>::value];
  int phase = 0;
  const bool is_log = (flags & kSoftmaxLog) != 0;
  const bool is_safe = (flags & kSoftmaxSafe) != 0;
  const int64_t xtiles = (((inner + E - 1) / E) + (1 << lay.tx_log2) - 1) >> lay.tx_log2;
  const int64_t ntiles = outer * xtiles;
  const int NG = groups_per_block<BLOCK>(lay);
  for (int64_t t0 = (int64_t)blockIdx.x * NG; t0 < ntiles; t0 += (int64_t)gridDim.x * NG) {
    const StridedTile tile = strided_tile<BLOCK, E>(t0, ntiles, xtiles, D, inner, lay);
    const int ty = tile.ty, TY = tile.TY;
    const TI* xs = x + tile.slab;
    TO* ys = y + tile.slab;
    float mx[E], sum[E];
#pragma unroll
    for (int i = 0; i < E; ++i) mx[i] = -INFINITY;
    for (int d = ty; d < D; d += TY) {
      const Pack<TI, E> p =
          load_row_pack<TI, E, false>(xs + (int64_t)d * inner, tile.e0, inner, tile.valid, -INFINITY);
#pragma unroll
      for (int i = 0; i < E; ++i) mx[i] = fmaxf(mx[i], p.get(i));
    }
    column_allreduce<BLOCK, E, MaxOp>(mx, lay, red, phase);
#pragma unroll
    for (int i = 0; i < E; ++i) sum[i] = 0.0f;
    for (int d = ty; d < D; d += TY) {
      const Pack<TI, E> p =
          load_row_pack<TI, E, false>(xs + (int64_t)d * inner, tile.e0, inner, tile.valid, -INFINITY);
#pragma unroll
      for (int i = 0; i < E; ++i) sum[i] += row_exp<PRECISE>(p.get(i) - mx[i]);
    }
    column_allreduce<BLOCK, E, SumOp>(sum, lay, red, phase);
    float kf[E];
#pragma unroll
    for (int i = 0; i < E; ++i) kf[i] = is_log ? logf(sum[i]) : 1.0f / sum[i];
    for (int d = ty; d < D; d += TY) {
      const Pack<TI, E> p =
          load_row_pack<TI, E, true>(xs + (int64_t)d * inner, tile.e0, inner, tile.valid, -INFINITY);
      Pack<TO, E> o;
      if (is_log) {
        ROWNORM_UNIFORM_ARM("log_softmax");
#pragma unroll
        for (int i = 0; i < E; ++i) o.set(i, (p.get(i) - mx[i]) - kf[i]);
      } else {
        ROWNORM_UNIFORM_ARM("softmax");
#pragma unroll
        for (int i = 0; i < E; ++i) {
          const float v = row_exp<PRECISE>(p.get(i) - mx[i]) * kf[i];
          o.set(i, (is_safe && mx[i] == -INFINITY) ? 0.0f : v);
        }
      }
      store_row_pack<TO, E, true>(ys + (int64_t)d * inner, tile.e0, inner, tile.valid, o);
    }
  }
}

template <class TG, class TO, int BLOCK>
__global__ void __launch_bounds__(BLOCK)
softmax_strided_bwd_stream_kernel(const TG* __restrict__ grad, const TG* __restrict__ y,
                                  TO* __restrict__ gi, int64_t outer, int D, int inner,
                                  StridedLayout lay, int flags) {
  constexpr int E = elems_per_pack<TG>::value;
  constexpr bool PRECISE = sizeof(TO) == 4 && sizeof(TG) == 4;
  __shared__ float red[column_lds_floats<BLOCK, E>::value];
  int phase = 0;
  const bool is_log = (flags & kSoftmaxLog) != 0;
  const int64_t xtiles = (((inner + E - 1) / E) + (1 << lay.tx_log2) - 1) >> lay.tx_log2;
  const int64_t ntiles = outer * xtiles;
  const int NG = groups_per_block<BLOCK>(lay);
  for (int64_t t0 = (int64_t)blockIdx.x * NG; t0 < ntiles; t0 += (int64_t)gridDim.x * NG) {
    const StridedTile tile = strided_tile<BLOCK, E>(t0, ntiles, xtiles, D, inner, lay);
    const int ty = tile.ty, TY = tile.TY;
    const TG* gs = grad + tile.slab;
    const TG* ys = y + tile.slab;
    TO* os = gi + tile.slab;
    float sum[E];
#pragma unroll
    for (int i = 0; i < E; ++i) sum[i] = 0.0f;
    for (int d = ty; d < D; d += TY) {
      const int64_t off = (int64_t)d * inner;
      const Pack<TG, E> pg = load_row_pack<TG, E, false>(gs + off, tile.e0, inner, tile.valid, 0.0f);
      if (is_log) {
#pragma unroll
        for (int i = 0; i < E; ++i) sum[i] += pg.get(i);
      } else {
        const Pack<TG, E> py = load_row_pack<TG, E, false>(ys + off, tile.e0, inner, tile.valid, 0.0f);
#pragma unroll
        for (int i = 0; i < E; ++i) sum[i] = fmaf(py.get(i), pg.get(i), sum[i]);
      }
    }
    column_allreduce<BLOCK, E, SumOp>(sum, lay, red, phase);
    for (int d = ty; d < D; d += TY) {
      const int64_t off = (int64_t)d * inner;
      const Pack<TG, E> pg = load_row_pack<TG, E, true>(gs + off, tile.e0, inner, tile.valid, 0.0f);
      const Pack<TG, E> py = load_row_pack<TG, E, true>(ys + off, tile.e0, inner, tile.valid, 0.0f);
      Pack<TO, E> o;
      if (is_log) {
        ROWNORM_UNIFORM_ARM("log_softmax backward");
#pragma unroll
        for (int i = 0; i < E; ++i) o.set(i, pg.get(i) - row_exp<PRECISE>(py.get(i)) * sum[i]);
      } else {
        ROWNORM_UNIFORM_ARM("softmax backward");
#pragma unroll
        for (int i = 0; i < E; ++i) o.set(i, py.get(i) * (pg.get(i) - sum[i]));
      }
      store_row_pack<TO, E, true>(os + off, tile.e0, inner, tile.valid, o);
    }
  }
}

// ---------------------------------------------------------------------------
// Large D with few columns' worth of tiles (softmax over dim 0 of an [8192, 8192]
// matrix is 128 tiles of 8192 rows): the D rows are cut into chunks so that the
// whole machine works, in three launches.
//
//   1. workgroup (tile, chunk) walks the rows of its chunk once and leaves, per
//      column, the running maximum m and the sum of exp(x - m) (forward), or the
//      sum of y * grad / grad (backward);
//   2. one workgroup a tile merges the chunks' values per column in a fixed order
//      -- M = max m_c, S = sum s_c * exp(m_c - M) -- and hands every chunk the
//      result;
//   3. workgroup (tile, chunk) reads the result and writes its rows.
//
// X is read twice (the second time from the last-level cache when the tensor
// fits it), Y written once; the multi-pass kernels above read X three times with
// one workgroup a tile.  The per-column values cross the launches inside the
// OUTPUT tensor, in the first rows of the chunk's own piece and in the columns
// they belong to -- memory that only workgroup (tile, chunk) of the third launch
// writes, after it has read them: no workspace, no allocation, and no workgroup
// waits for another.  NF floats a column (2 forward, 1 backward) take
// NF * 4 / sizeof(TO) rows: the 32-bit patterns are cut into pieces of the
// output's element size, so that the pack accessors (ragged `inner`, any
// alignment) move them like data.  The output must not overlap an input.
template <class TO, int NF>
struct split_slot_rows {
  static constexpr int value = NF * 4 / (int)sizeof(TO);
};

template <class TO, int E, int NF>
__device__ __forceinline__ void split_slot_store(TO* row0, int inner, int e0, bool valid,
                                                 const float (&a)[E], const float (&b)[E]) {
  constexpr int R = split_slot_rows<TO, NF>::value;
#pragma unroll
  for (int r = 0; r < R; ++r) {
    Pack<TO, E> p;
#pragma unroll
    for (int i = 0; i < E; ++i) {
      if constexpr (sizeof(TO) == 4) {
        p.v[i] = __builtin_bit_cast(TO, r == 0 ? a[i] : b[i]);
      } else {
        const uint32_t w = __builtin_bit_cast(uint32_t, r < 2 ? a[i] : b[i]);
        p.v[i] = __builtin_bit_cast(TO, (uint16_t)((r & 1) ? (w >> 16) : (w & 0xffffu)));
      }
    }
    store_row_pack<TO, E, false>(row0 + (int64_t)r * inner, e0, inner, valid, p);
  }
}

template <class TO, int E, int NF>
__device__ __forceinline__ void split_slot_load(const TO* row0, int inner, int e0, bool valid,
                                                float (&a)[E], float (&b)[E]) {
  constexpr int R = split_slot_rows<TO, NF>::value;
  Pack<TO, E> p[R];
#pragma unroll
  for (int r = 0; r < R; ++r)
    p[r] = load_row_pack<TO, E, false>(row0 + (int64_t)r * inner, e0, inner, valid, 0.0f);
  // (each element is copied into a plain variable first: a bit cast applied to an
  // element of a vector directly reads the vector's first element)
#pragma unroll
  for (int i = 0; i < E; ++i) {
    TO t[R];
#pragma unroll
    for (int r = 0; r < R; ++r) t[r] = p[r].v[i];
    if constexpr (sizeof(TO) == 4) {
      a[i] = __builtin_bit_cast(float, t[0]);
      b[i] = NF == 2 ? __builtin_bit_cast(float, t[NF - 1]) : 0.0f;
    } else {
      const uint32_t lo = __builtin_bit_cast(uint16_t, t[0]);
      const uint32_t hi = __builtin_bit_cast(uint16_t, t[1]);
      a[i] = __builtin_bit_cast(float, lo | (hi << 16));
      if constexpr (NF == 2) {
        const uint32_t lo2 = __builtin_bit_cast(uint16_t, t[R - 2]);
        const uint32_t hi2 = __builtin_bit_cast(uint16_t, t[R - 1]);
        b[i] = __builtin_bit_cast(float, lo2 | (hi2 << 16));
      } else {
        b[i] = 0.0f;
      }
    }
  }
}

// Rows [d0, d1) of chunk `c` out of `chunks` (the last chunk takes the remainder).
__device__ __forceinline__ void split_rows(int c, int chunks, int chunk_rows, int D, int* d0,
                                           int* d1) {
  *d0 = c * chunk_rows;
  *d1 = c == chunks - 1 ? D : *d0 + chunk_rows;
}

// Merges (m, s) pairs: the running maximum and the sum of exp(x - maximum).
template <bool PRECISE>
__device__ __forceinline__ void online_merge(float& m, float& s, float m2, float s2) {
  const float nm = fmaxf(m, m2);
  if (nm != -INFINITY)  // (both empty: nothing to rescale, and -inf - -inf is NaN)
    s = s * row_exp<PRECISE>(m - nm) + s2 * row_exp<PRECISE>(m2 - nm);
  else
    s = s + s2;  // 0 + 0, or NaN if an operand carries one
  m = nm;
}

// After a lane has walked its rows: the group's (M, S) per column, in every lane.
template <int BLOCK, int E, bool PRECISE>
__device__ __forceinline__ void column_merge_online(float (&mx)[E], float (&sum)[E],
                                                    StridedLayout lay, float* lds, int& phase) {
  float mall[E];
#pragma unroll
  for (int i = 0; i < E; ++i) mall[i] = mx[i];
  column_allreduce<BLOCK, E, MaxOp>(mall, lay, lds, phase);
#pragma unroll
  for (int i = 0; i < E; ++i) {
    sum[i] = mall[i] != -INFINITY ? sum[i] * row_exp<PRECISE>(mx[i] - mall[i]) : sum[i];
    mx[i] = mall[i];
  }
  column_allreduce<BLOCK, E, SumOp>(sum, lay, lds, phase);
}

constexpr int kSplitUnroll = 4;  // rows a lane requests before it uses any of them

// Launch 1, forward.  grid (blocks over tiles, chunks).
template <class TI, class TO, int BLOCK>
__global__ void __launch_bounds__(BLOCK)
softmax_strided_split_partial_kernel(const TI* __restrict__ x, TO* __restrict__ y, int64_t outer,
                                     int D, int inner, StridedLayout lay, int chunk_rows) {
  constexpr int E = elems_per_pack<TI>::value;
  constexpr bool PRECISE = sizeof(TO) == 4;
  constexpr int U = kSplitUnroll;
  __shared__ float red[column_lds_floats<BLOCK, E>::value];
  int phase = 0;
  const int64_t xtiles = (((inner + E - 1) / E) + (1 << lay.tx_log2) - 1) >> lay.tx_log2;
  const int64_t ntiles = outer * xtiles;
  const int NG = groups_per_block<BLOCK>(lay);
  int d0, d1;
  split_rows(blockIdx.y, gridDim.y, chunk_rows, D, &d0, &d1);
  for (int64_t t0 = (int64_t)blockIdx.x * NG; t0 < ntiles; t0 += (int64_t)gridDim.x * NG) {
    const StridedTile tile = strided_tile<BLOCK, E>(t0, ntiles, xtiles, D, inner, lay);
    const int ty = tile.ty, TY = tile.TY;
    const TI* xs = x + tile.slab;
    float mx[E], sum[E];
#pragma unroll
    for (int i = 0; i < E; ++i) {
      mx[i] = -INFINITY;
      sum[i] = 0.0f;
    }
    for (int d = d0 + ty; d < d1; d += TY * U) {
      Pack<TI, E> p[U];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int dd = d + u * TY;
        const bool ok = tile.valid && dd < d1;
        p[u] = load_row_pack<TI, E, false>(xs + (int64_t)(ok ? dd : d0) * inner, tile.e0, inner,
                                           ok, -INFINITY);
      }
#pragma unroll
      for (int i = 0; i < E; ++i) {
        float nm = mx[i];
#pragma unroll
        for (int u = 0; u < U; ++u) nm = fmaxf(nm, p[u].get(i));
        // (no branch: while nothing finite has been seen the reference is 0, against
        // which -inf elements add 0 and a NaN element, which fmaxf drops, still poisons
        // the sum)
        const float ref = nm == -INFINITY ? 0.0f : nm;
        float acc = sum[i] * row_exp<PRECISE>(mx[i] - ref);
#pragma unroll
        for (int u = 0; u < U; ++u) acc += row_exp<PRECISE>(p[u].get(i) - ref);
        sum[i] = acc;
        mx[i] = nm;
      }
    }
    column_merge_online<BLOCK, E, PRECISE>(mx, sum, lay, red, phase);
    if (ty == 0)
      split_slot_store<TO, E, 2>(y + tile.slab + (int64_t)d0 * inner, inner, tile.e0, tile.valid,
                                 mx, sum);
  }
}

// Launch 2 (forward and backward): one group a tile; lane (ty, tx) takes the chunks
// ty, ty + TY, ... of its columns, the group merges them, and each lane writes the
// result back over the chunks it read.  NF = 2: (m, s) pairs; NF = 1: plain sums.
template <class TO, int E, int NF, int BLOCK>
__global__ void __launch_bounds__(BLOCK)
softmax_strided_split_combine_kernel(TO* __restrict__ y, int64_t outer, int D, int inner,
                                     StridedLayout lay, int chunk_rows, int chunks) {
  constexpr bool PRECISE = sizeof(TO) == 4;
  __shared__ float red[column_lds_floats<BLOCK, E>::value];
  int phase = 0;
  const int64_t xtiles = (((inner + E - 1) / E) + (1 << lay.tx_log2) - 1) >> lay.tx_log2;
  const int64_t ntiles = outer * xtiles;
  const int NG = groups_per_block<BLOCK>(lay);
  for (int64_t t0 = (int64_t)blockIdx.x * NG; t0 < ntiles; t0 += (int64_t)gridDim.x * NG) {
    const StridedTile tile = strided_tile<BLOCK, E>(t0, ntiles, xtiles, D, inner, lay);
    const int ty = tile.ty, TY = tile.TY;
    TO* ys = y + tile.slab;
    float a[E], b[E];
#pragma unroll
    for (int i = 0; i < E; ++i) {
      a[i] = NF == 2 ? -INFINITY : 0.0f;
      b[i] = 0.0f;
    }
    for (int c = ty; c < chunks; c += TY) {
      float ca[E], cb[E];
      split_slot_load<TO, E, NF>(ys + (int64_t)c * chunk_rows * inner, inner, tile.e0, tile.valid,
                                 ca, cb);
#pragma unroll
      for (int i = 0; i < E; ++i) {
        if constexpr (NF == 2)
          online_merge<PRECISE>(a[i], b[i], ca[i], cb[i]);
        else
          a[i] += ca[i];
      }
    }
    if constexpr (NF == 2)
      column_merge_online<BLOCK, E, PRECISE>(a, b, lay, red, phase);
    else
      column_allreduce<BLOCK, E, SumOp>(a, lay, red, phase);
    for (int c = ty; c < chunks; c += TY)
      split_slot_store<TO, E, NF>(ys + (int64_t)c * chunk_rows * inner, inner, tile.e0, tile.valid,
                                  a, b);
  }
}

// Launch 3, forward.
template <class TI, class TO, int BLOCK>
__global__ void __launch_bounds__(BLOCK)
softmax_strided_split_apply_kernel(const TI* __restrict__ x, TO* __restrict__ y, int64_t outer,
                                   int D, int inner, StridedLayout lay, int chunk_rows,
                                   int flags) {
  constexpr int E = elems_per_pack<TI>::value;
  constexpr bool PRECISE = sizeof(TO) == 4;
  constexpr int U = kSplitUnroll;
  const bool is_log = (flags & kSoftmaxLog) != 0;
  const bool is_safe = (flags & kSoftmaxSafe) != 0;
  const int64_t xtiles = (((inner + E - 1) / E) + (1 << lay.tx_log2) - 1) >> lay.tx_log2;
  const int64_t ntiles = outer * xtiles;
  const int NG = groups_per_block<BLOCK>(lay);
  int d0, d1;
  split_rows(blockIdx.y, gridDim.y, chunk_rows, D, &d0, &d1);
  for (int64_t t0 = (int64_t)blockIdx.x * NG; t0 < ntiles; t0 += (int64_t)gridDim.x * NG) {
    const StridedTile tile = strided_tile<BLOCK, E>(t0, ntiles, xtiles, D, inner, lay);
    const int ty = tile.ty, TY = tile.TY;
    const TI* xs = x + tile.slab;
    TO* ys = y + tile.slab;
    float mx[E], sum[E], kf[E];
    split_slot_load<TO, E, 2>(ys + (int64_t)d0 * inner, inner, tile.e0, tile.valid, mx, sum);
    __syncthreads();  // every lane has its columns' (M, S) before the rows that hold them are written
#pragma unroll
    for (int i = 0; i < E; ++i) kf[i] = is_log ? logf(sum[i]) : 1.0f / sum[i];
    for (int d = d0 + ty; d < d1; d += TY * U) {
      Pack<TI, E> p[U];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int dd = d + u * TY;
        const bool ok = tile.valid && dd < d1;
        p[u] = load_row_pack<TI, E, true>(xs + (int64_t)(ok ? dd : d0) * inner, tile.e0, inner, ok,
                                          -INFINITY);
      }
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int dd = d + u * TY;
        const bool ok = tile.valid && dd < d1;
        Pack<TO, E> o;
        if (is_log) {
          ROWNORM_UNIFORM_ARM("log_softmax, rows split over workgroups");
#pragma unroll
          for (int i = 0; i < E; ++i) o.set(i, (p[u].get(i) - mx[i]) - kf[i]);
        } else {
          ROWNORM_UNIFORM_ARM("softmax, rows split over workgroups");
#pragma unroll
          for (int i = 0; i < E; ++i) {
            const float v = row_exp<PRECISE>(p[u].get(i) - mx[i]) * kf[i];
            o.set(i, (is_safe && mx[i] == -INFINITY) ? 0.0f : v);
          }
        }
        store_row_pack<TO, E, true>(ys + (int64_t)(ok ? dd : d0) * inner, tile.e0, inner, ok, o);
      }
    }
  }
}

// Launch 1, backward: the chunk's sum of y * grad (softmax) or grad (log_softmax).
template <class TG, class TO, int BLOCK>
__global__ void __launch_bounds__(BLOCK)
softmax_strided_split_bwd_partial_kernel(const TG* __restrict__ grad, const TG* __restrict__ y,
                                         TO* __restrict__ gi, int64_t outer, int D, int inner,
                                         StridedLayout lay, int chunk_rows, int flags) {
  constexpr int E = elems_per_pack<TG>::value;
  constexpr int U = kSplitUnroll;
  __shared__ float red[column_lds_floats<BLOCK, E>::value];
  int phase = 0;
  const bool is_log = (flags & kSoftmaxLog) != 0;
  const int64_t xtiles = (((inner + E - 1) / E) + (1 << lay.tx_log2) - 1) >> lay.tx_log2;
  const int64_t ntiles = outer * xtiles;
  const int NG = groups_per_block<BLOCK>(lay);
  int d0, d1;
  split_rows(blockIdx.y, gridDim.y, chunk_rows, D, &d0, &d1);
  for (int64_t t0 = (int64_t)blockIdx.x * NG; t0 < ntiles; t0 += (int64_t)gridDim.x * NG) {
    const StridedTile tile = strided_tile<BLOCK, E>(t0, ntiles, xtiles, D, inner, lay);
    const int ty = tile.ty, TY = tile.TY;
    const TG* gs = grad + tile.slab;
    const TG* ys = y + tile.slab;
    float sum[E], unused[E];
#pragma unroll
    for (int i = 0; i < E; ++i) sum[i] = unused[i] = 0.0f;
    // (one loop per variant: a test of the variant around the load of y inside the loop
    // is a branch whose join waits for every request outstanding, which made the 2 * U
    // loads of an iteration complete one after the other)
    auto add_rows = [&](auto log_variant) {
      constexpr bool LOG = decltype(log_variant)::value;
      for (int d = d0 + ty; d < d1; d += TY * U) {
        Pack<TG, E> pg[U], py[LOG ? 1 : U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
          const int dd = d + u * TY;
          const bool ok = tile.valid && dd < d1;
          const int64_t off = (int64_t)(ok ? dd : d0) * inner;
          pg[u] = load_row_pack<TG, E, false>(gs + off, tile.e0, inner, ok, 0.0f);
          if constexpr (!LOG)
            py[u] = load_row_pack<TG, E, false>(ys + off, tile.e0, inner, ok, 0.0f);
        }
#pragma unroll
        for (int u = 0; u < U; ++u)
#pragma unroll
          for (int i = 0; i < E; ++i)
            sum[i] = LOG ? sum[i] + pg[u].get(i)
                         : fmaf(py[LOG ? 0 : u].get(i), pg[u].get(i), sum[i]);
      }
    };
    if (is_log)
      add_rows(std::true_type{});
    else
      add_rows(std::false_type{});
    column_allreduce<BLOCK, E, SumOp>(sum, lay, red, phase);
    if (ty == 0)
      split_slot_store<TO, E, 1>(gi + tile.slab + (int64_t)d0 * inner, inner, tile.e0, tile.valid,
                                 sum, unused);
  }
}

// Launch 3, backward.
template <class TG, class TO, int BLOCK>
__global__ void __launch_bounds__(BLOCK)
softmax_strided_split_bwd_apply_kernel(const TG* __restrict__ grad, const TG* __restrict__ y,
                                       TO* __restrict__ gi, int64_t outer, int D, int inner,
                                       StridedLayout lay, int chunk_rows, int flags) {
  constexpr int E = elems_per_pack<TG>::value;
  constexpr bool PRECISE = sizeof(TO) == 4 && sizeof(TG) == 4;
  constexpr int U = kSplitUnroll;
  const bool is_log = (flags & kSoftmaxLog) != 0;
  const int64_t xtiles = (((inner + E - 1) / E) + (1 << lay.tx_log2) - 1) >> lay.tx_log2;
  const int64_t ntiles = outer * xtiles;
  const int NG = groups_per_block<BLOCK>(lay);
  int d0, d1;
  split_rows(blockIdx.y, gridDim.y, chunk_rows, D, &d0, &d1);
  for (int64_t t0 = (int64_t)blockIdx.x * NG; t0 < ntiles; t0 += (int64_t)gridDim.x * NG) {
    const StridedTile tile = strided_tile<BLOCK, E>(t0, ntiles, xtiles, D, inner, lay);
    const int ty = tile.ty, TY = tile.TY;
    const TG* gs = grad + tile.slab;
    const TG* ys = y + tile.slab;
    TO* os = gi + tile.slab;
    float sum[E], unused[E];
    split_slot_load<TO, E, 1>(os + (int64_t)d0 * inner, inner, tile.e0, tile.valid, sum, unused);
    __syncthreads();  // the sums are read before the rows that hold them are written
    for (int d = d0 + ty; d < d1; d += TY * U) {
      Pack<TG, E> pg[U], py[U];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int dd = d + u * TY;
        const bool ok = tile.valid && dd < d1;
        const int64_t off = (int64_t)(ok ? dd : d0) * inner;
        pg[u] = load_row_pack<TG, E, true>(gs + off, tile.e0, inner, ok, 0.0f);
        py[u] = load_row_pack<TG, E, true>(ys + off, tile.e0, inner, ok, 0.0f);
      }
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int dd = d + u * TY;
        const bool ok = tile.valid && dd < d1;
        Pack<TO, E> o;
        if (is_log) {
          ROWNORM_UNIFORM_ARM("log_softmax backward, rows split over workgroups");
#pragma unroll
          for (int i = 0; i < E; ++i)
            o.set(i, pg[u].get(i) - row_exp<PRECISE>(py[u].get(i)) * sum[i]);
        } else {
          ROWNORM_UNIFORM_ARM("softmax backward, rows split over workgroups");
#pragma unroll
          for (int i = 0; i < E; ++i) o.set(i, py[u].get(i) * (pg[u].get(i) - sum[i]));
        }
        store_row_pack<TO, E, true>(os + (int64_t)(ok ? dd : d0) * inner, tile.e0, inner, ok, o);
      }
    }
  }
}

}  // namespace rownorm
