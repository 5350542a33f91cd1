// Last-dimension softmax / log_softmax forward and backward for gfx950.
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
#pragma once
#include "device/pack.hpp"
#include "device/reduce.hpp"

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

template <class TI, class TO, int G, int V, int BLOCK, bool FAST>
__global__ void __launch_bounds__(BLOCK)
softmax_fwd_resident_kernel(const TI* __restrict__ x, TO* __restrict__ y, int64_t M, int N,
                            int is_log) {
  constexpr int E = elems_per_pack<TI>::value;
  constexpr int RPB = BLOCK / G;
  constexpr bool PRECISE = sizeof(TO) == 4;
  __shared__ float red[reduce_lds_floats<G, BLOCK, 1>::value];
  int phase = 0;
  const int slot = threadIdx.x / G;
  const int lane = threadIdx.x % G;
  const int64_t nrb = (M + RPB - 1) / RPB;
  for (int64_t rb = blockIdx.x; rb < nrb; rb += gridDim.x) {
    const int64_t row = rb * RPB + slot;
    const bool ok = RPB == 1 ? true : row < M;
    const TI* xr = x + (ok ? row : 0) * (int64_t)N;
    TO* yr = y + row * (int64_t)N;
    Pack<TI, E> xp[V];
#pragma unroll
    for (int c = 0; c < V; ++c)
      xp[c] = row_load<TI, E, true, FAST>(xr, (c * G + lane) * E, N, ok, -INFINITY);
    float xf[V][E];
#pragma unroll
    for (int c = 0; c < V; ++c)
#pragma unroll
      for (int i = 0; i < E; ++i) xf[c][i] = xp[c].get(i);
    float mx[1] = {-INFINITY};
#pragma unroll
    for (int c = 0; c < V; ++c)
#pragma unroll
      for (int i = 0; i < E; ++i) mx[0] = fmaxf(mx[0], xf[c][i]);
    group_allreduce<G, BLOCK, 1, MaxOp>(mx, red, phase);
    const float m = mx[0];
    float sum[1] = {0.0f};
    if (is_log) {
      // keep x - m; the exponentials are only needed for the sum
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
    const float k = is_log ? logf(sum[0]) : 1.0f / sum[0];
#pragma unroll
    for (int c = 0; c < V; ++c) {
      const int e0 = (c * G + lane) * E;
      Pack<TO, E> o;
#pragma unroll
      for (int i = 0; i < E; ++i) o.set(i, is_log ? xf[c][i] - k : xf[c][i] * k);
      row_store<TO, E, true, FAST>(yr, e0, N, ok, o);
    }
  }
}

// Rows too wide for registers: one workgroup per row, three streaming passes.
template <class TI, class TO, int BLOCK>
__global__ void __launch_bounds__(BLOCK)
softmax_fwd_stream_kernel(const TI* __restrict__ x, TO* __restrict__ y, int64_t M, int N,
                          int is_log) {
  constexpr int E = elems_per_pack<TI>::value;
  constexpr bool PRECISE = sizeof(TO) == 4;
  __shared__ float red[reduce_lds_floats<BLOCK, BLOCK, 1>::value];
  int phase = 0;
  const int npacks = (N + E - 1) / E;
  for (int64_t row = blockIdx.x; row < M; row += gridDim.x) {
    const TI* xr = x + row * (int64_t)N;
    TO* yr = y + row * (int64_t)N;
    float mx[1] = {-INFINITY};
    for (int pk = threadIdx.x; pk < npacks; pk += BLOCK) {
      const Pack<TI, E> p = load_row_pack<TI, E, false>(xr, pk * E, N, true, -INFINITY);
#pragma unroll
      for (int i = 0; i < E; ++i) mx[0] = fmaxf(mx[0], p.get(i));
    }
    group_allreduce<BLOCK, BLOCK, 1, MaxOp>(mx, red, phase);
    const float m = mx[0];
    float sum[1] = {0.0f};
    for (int pk = threadIdx.x; pk < npacks; pk += BLOCK) {
      const Pack<TI, E> p = load_row_pack<TI, E, false>(xr, pk * E, N, true, -INFINITY);
#pragma unroll
      for (int i = 0; i < E; ++i) sum[0] += row_exp<PRECISE>(p.get(i) - m);
    }
    group_allreduce<BLOCK, BLOCK, 1, SumOp>(sum, red, phase);
    const float k = is_log ? logf(sum[0]) : 1.0f / sum[0];
    for (int pk = threadIdx.x; pk < npacks; pk += BLOCK) {
      const int e0 = pk * E;
      const Pack<TI, E> p = load_row_pack<TI, E, true>(xr, e0, N, true, -INFINITY);
      Pack<TO, E> o;
#pragma unroll
      for (int i = 0; i < E; ++i) {
        const float d = p.get(i) - m;
        o.set(i, is_log ? d - k : row_exp<PRECISE>(d) * k);
      }
      store_row_pack<TO, E, true>(yr, e0, N, true, o);
    }
  }
}

// Backward.  TG: dtype of grad and of y (the saved forward output); TO: dtype
// of the input gradient.
template <class TG, class TO, int G, int V, int BLOCK, bool FAST>
__global__ void __launch_bounds__(BLOCK)
softmax_bwd_resident_kernel(const TG* __restrict__ grad, const TG* __restrict__ y,
                            TO* __restrict__ gi, int64_t M, int N, int is_log) {
  constexpr int E = elems_per_pack<TG>::value;
  constexpr int RPB = BLOCK / G;
  constexpr bool PRECISE = sizeof(TO) == 4 && sizeof(TG) == 4;
  __shared__ float red[reduce_lds_floats<G, BLOCK, 1>::value];
  int phase = 0;
  const int slot = threadIdx.x / G;
  const int lane = threadIdx.x % G;
  const int64_t nrb = (M + RPB - 1) / RPB;
  for (int64_t rb = blockIdx.x; rb < nrb; rb += gridDim.x) {
    const int64_t row = rb * RPB + slot;
    const bool ok = RPB == 1 ? true : row < M;
    const int64_t rowc = ok ? row : 0;
    const TG* gr = grad + rowc * (int64_t)N;
    const TG* yr = y + rowc * (int64_t)N;
    TO* outr = gi + row * (int64_t)N;
    Pack<TG, E> pg[V], py[V];
#pragma unroll
    for (int c = 0; c < V; ++c) {
      const int e0 = (c * G + lane) * E;
      pg[c] = row_load<TG, E, true, FAST>(gr, e0, N, ok, 0.0f);
      py[c] = row_load<TG, E, true, FAST>(yr, e0, N, ok, 0.0f);
    }
    float gf[V][E], yf[V][E];
#pragma unroll
    for (int c = 0; c < V; ++c)
#pragma unroll
      for (int i = 0; i < E; ++i) {
        gf[c][i] = pg[c].get(i);
        yf[c][i] = py[c].get(i);
      }
    float sum[1] = {0.0f};
    if (is_log) {
#pragma unroll
      for (int c = 0; c < V; ++c)
#pragma unroll
        for (int i = 0; i < E; ++i) sum[0] += gf[c][i];
    } else {
#pragma unroll
      for (int c = 0; c < V; ++c)
#pragma unroll
        for (int i = 0; i < E; ++i) sum[0] = fmaf(yf[c][i], gf[c][i], sum[0]);
    }
    group_allreduce<G, BLOCK, 1, SumOp>(sum, red, phase);
    const float s = sum[0];
#pragma unroll
    for (int c = 0; c < V; ++c) {
      const int e0 = (c * G + lane) * E;
      Pack<TO, E> o;
#pragma unroll
      for (int i = 0; i < E; ++i) {
        const float v = is_log ? gf[c][i] - row_exp<PRECISE>(yf[c][i]) * s
                               : yf[c][i] * (gf[c][i] - s);
        o.set(i, v);
      }
      row_store<TO, E, true, FAST>(outr, e0, N, ok, o);
    }
  }
}

template <class TG, class TO, int BLOCK>
__global__ void __launch_bounds__(BLOCK)
softmax_bwd_stream_kernel(const TG* __restrict__ grad, const TG* __restrict__ y,
                          TO* __restrict__ gi, int64_t M, int N, int is_log) {
  constexpr int E = elems_per_pack<TG>::value;
  constexpr bool PRECISE = sizeof(TO) == 4 && sizeof(TG) == 4;
  __shared__ float red[reduce_lds_floats<BLOCK, BLOCK, 1>::value];
  int phase = 0;
  const int npacks = (N + E - 1) / E;
  for (int64_t row = blockIdx.x; row < M; row += gridDim.x) {
    const TG* gr = grad + row * (int64_t)N;
    const TG* yr = y + row * (int64_t)N;
    TO* outr = gi + row * (int64_t)N;
    float sum[1] = {0.0f};
    for (int pk = threadIdx.x; pk < npacks; pk += BLOCK) {
      const Pack<TG, E> pg = load_row_pack<TG, E, false>(gr, pk * E, N, true, 0.0f);
      if (is_log) {
#pragma unroll
        for (int i = 0; i < E; ++i) sum[0] += pg.get(i);
      } else {
        const Pack<TG, E> py = load_row_pack<TG, E, false>(yr, pk * E, N, true, 0.0f);
#pragma unroll
        for (int i = 0; i < E; ++i) sum[0] = fmaf(py.get(i), pg.get(i), sum[0]);
      }
    }
    group_allreduce<BLOCK, BLOCK, 1, SumOp>(sum, red, phase);
    const float s = sum[0];
    for (int pk = threadIdx.x; pk < npacks; pk += BLOCK) {
      const int e0 = pk * E;
      const Pack<TG, E> pg = load_row_pack<TG, E, true>(gr, e0, N, true, 0.0f);
      const Pack<TG, E> py = load_row_pack<TG, E, true>(yr, e0, N, true, 0.0f);
      Pack<TO, E> o;
#pragma unroll
      for (int i = 0; i < E; ++i) {
        const float v = is_log ? pg.get(i) - row_exp<PRECISE>(py.get(i)) * s
                               : py.get(i) * (pg.get(i) - s);
        o.set(i, v);
      }
      store_row_pack<TO, E, true>(outr, e0, N, true, o);
    }
  }
}

}  // namespace rownorm
