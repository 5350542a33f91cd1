// All-reduce of a few fp32 values over the G lanes that share one row.
//
// G <= 64: the lanes sit in one wavefront.  Four DPP steps (quad_perm xor 1,
// xor 2, row_half_mirror, row_mirror) leave the 16-lane sums in every lane of
// each DPP row; the four row values are then read through v_readlane and
// combined, so every lane ends with the result and no broadcast step exists.
// G > 64: each wavefront reduces as above, lane 0 parks the wave value in
// LDS, one barrier, and every lane sums the G/64 parked values in a fixed
// order (deterministic).  The LDS area is double buffered by the caller-held
// phase bit, so consecutive reductions need one barrier each.
//
// Role in the reference: norm_group_reduce (src/ATen/native/xpu/sycl/Norm.h:
// 38-106), softmax_group_reduce (SoftMaxKernels.cpp:39-102) and
// GroupReduceWithoutBroadcast (GroupReduceUtils.h), which shuffle down to one
// lane, go through local memory and broadcast back.
#pragma once
#include <hip/hip_runtime.h>

namespace rownorm {

struct SumOp {
  __device__ __forceinline__ static float apply(float a, float b) { return a + b; }
  __device__ __forceinline__ static float identity() { return 0.0f; }
};
struct MaxOp {
  // v_max_f32 drops a NaN operand.  That is harmless for softmax: a NaN element
  // still turns exp(x - max) and therefore the row sum into NaN, so the whole
  // row comes out NaN either way.
  __device__ __forceinline__ static float apply(float a, float b) { return fmaxf(a, b); }
  __device__ __forceinline__ static float identity() { return -INFINITY; }
};

template <int CTRL>
__device__ __forceinline__ float dpp_move(float v) {
  return __builtin_bit_cast(
      float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, true));
}

__device__ __forceinline__ float read_lane(float v, int lane) {
  return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), lane));
}

// Reduction over aligned groups of G lanes (G in {1,2,4,8,16,32,64}) of one
// wavefront; the result is present in every lane of the group.
template <int G, class Op>
__device__ __forceinline__ float wave_group_allreduce(float v) {
  static_assert(G >= 1 && G <= 64 && (G & (G - 1)) == 0, "G must be a power of two <= 64");
  if constexpr (G >= 2) v = Op::apply(v, dpp_move<0xB1>(v));   // quad_perm [1,0,3,2]
  if constexpr (G >= 4) v = Op::apply(v, dpp_move<0x4E>(v));   // quad_perm [2,3,0,1]
  if constexpr (G >= 8) v = Op::apply(v, dpp_move<0x141>(v));  // row_half_mirror
  if constexpr (G >= 16) v = Op::apply(v, dpp_move<0x140>(v)); // row_mirror
  if constexpr (G >= 32) {
    const float r0 = read_lane(v, 0), r1 = read_lane(v, 16);
    const float r2 = read_lane(v, 32), r3 = read_lane(v, 48);
    const float lo = Op::apply(r0, r1), hi = Op::apply(r2, r3);
    if constexpr (G == 64) {
      v = Op::apply(lo, hi);
    } else {
      v = (threadIdx.x & 32) ? hi : lo;
    }
  }
  return v;
}

// LDS floats needed by group_allreduce for a block of BLOCK threads reducing K values.
template <int G, int BLOCK, int K>
struct reduce_lds_floats {
  static constexpr int value = (G > 64) ? 2 * (BLOCK / 64) * K : 1;
};

// All-reduce of K values over each group of G consecutive threads of the block.
// Every thread of the block must call it (it contains a barrier when G > 64).
template <int G, int BLOCK, int K, class Op>
__device__ __forceinline__ void group_allreduce(float (&v)[K], float* lds, int& phase) {
#pragma unroll
  for (int k = 0; k < K; ++k) v[k] = wave_group_allreduce<(G < 64 ? G : 64), Op>(v[k]);
  if constexpr (G > 64) {
    constexpr int WPG = G / 64;  // wavefronts per row group
    constexpr int NW = BLOCK / 64;
    const int wave = threadIdx.x >> 6;
    float* buf = lds + phase * (NW * K);
    if ((threadIdx.x & 63) == 0) {
#pragma unroll
      for (int k = 0; k < K; ++k) buf[wave * K + k] = v[k];
    }
    __syncthreads();
    const int w0 = (wave / WPG) * WPG;
#pragma unroll
    for (int k = 0; k < K; ++k) {
      float acc = buf[w0 * K + k];
#pragma unroll
      for (int w = 1; w < WPG; ++w) acc = Op::apply(acc, buf[(w0 + w) * K + k]);
      v[k] = acc;
    }
    phase ^= 1;
  }
}

// Sum of two float64 values per thread over the workgroup, added in a fixed
// order; the result is valid in thread 0 only.
template <int BLOCK>
__device__ __forceinline__ void block_sum2_f64(double& a, double& b, double* lds) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    a += __shfl_down(a, off, 64);
    b += __shfl_down(b, off, 64);
  }
  const int wave = threadIdx.x >> 6;
  if ((threadIdx.x & 63) == 0) {
    lds[2 * wave] = a;
    lds[2 * wave + 1] = b;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    a = lds[0];
    b = lds[1];
#pragma unroll
    for (int w = 1; w < BLOCK / 64; ++w) {
      a += lds[2 * w];
      b += lds[2 * w + 1];
    }
  }
}

// The per-row scalar arithmetic (sum / N, 1 / sqrt(var + eps)) is evaluated by
// every lane of the row, and an IEEE float32 division or square root is about
// ten VALU instructions: with 16 elements a lane, the two divisions, the square
// root and the reciprocal of a LayerNorm row were a sixth of all the vector
// instructions of the 16-bit forward, a kernel that runs the vector ALU at
// 60 % while it streams from HBM.  16-bit rows therefore multiply by 1 / N
// (rounded once, outside the row loop) and take the hardware reciprocal square
// root (v_rsq_f32, one ulp): both move mean / rstd by a float32 ulp, four
// orders of magnitude inside the 16-bit tolerance, and change nothing on a
// constant row (the sums are exactly zero there).  float32 rows keep the
// correctly rounded division and square root.
template <class T>
__device__ __forceinline__ float row_mean_of(float sum, float fN, float inv_n) {
  if constexpr (sizeof(T) == 2)
    return sum * inv_n;
  else
    return sum / fN;
}

template <class T>
__device__ __forceinline__ float row_rstd_of(float v) {
  if constexpr (sizeof(T) == 2)
    return __builtin_amdgcn_rsqf(v);
  else
    return 1.0f / sqrtf(v);
}

}  // namespace rownorm
