// Short rows staged through LDS: what the softmax and norm kernels for short ragged rows
// share (layout rule, staging, LDS row access).
#pragma once
#include <stdint.h>

#include "pack.hpp"
#include "../plan.hpp"

namespace rownorm {

// ---------------------------------------------------------------------------
// Short ragged rows (N % E != 0, N <= 64 lanes * kFlatMaxPacks packs: ViT / CLIP /
// Whisper attention scores are rows of 197, 577, 77, 1500 elements) through LDS.  Such
// rows start at every 2-byte (fp32: 4-byte) alignment, and the general kernels
// pay for it per row: edge packs moved element by element, windows, masks.  But
// a run of `chunk_rows` consecutive rows, chunk_rows a multiple of 8, is one
// contiguous piece of the tensor that starts and ends on a 16-byte boundary, so
// the workgroup copies the piece to LDS with whole aligned 128-bit accesses, each
// group of G lanes then reads a row from LDS in packs at the row's own alignment
// (LDS takes unaligned 128-bit accesses; VP packs a lane, laid out like the
// register-resident kernels'), writes the results back in place, and the piece
// leaves with whole 128-bit stores: HBM sees the access pattern of a copy
// whatever N is.  The reductions stay inside a wavefront (G <= 64), so the only
// barriers are the two around the LDS phase; a lane group walks the rows r,
// r + BLOCK / G, ... of the piece.  Needs 16-byte aligned tensor bases and the
// same dtype in and out; anything else keeps the general kernels.  Very short
// rows of whole packs whose pack count fits the resident layouts badly take the
// same path (flat_layout below).
constexpr int kFlatBlock = 256;
// LDS per tensor a workgroup holds (LDSB; the backward holds two tensors): 16 KB
// at 256 threads, so that 8 workgroups share a compute unit; the backward takes
// 8 KB per tensor where that still holds a full pass of rows, for the same
// reason; rows beyond 1024 16-bit elements need 32 KB to hold 8 of them.
// Measured against 512 threads / 32 KB: bf16 [151296, 197] forward 27.0 -> 25.6 us,
// backward 36.2 -> 32.9 us ([147712, 577] backward, which needs the 16 KB:
// 101 -> 94 us); 1024 threads were 50 % slower.
constexpr int kFlatLdsBytes = 64 * kFlatBlock;
// Lanes per row G (1..64) and packs per lane VP (1..kFlatMaxPacks) are chosen so
// that G * VP leaves as few pack slots idle as possible (flat_layout below).
constexpr int kFlatMaxPacks = 4;
// Rows a workgroup takes at a time: as many as its LDS holds, a multiple of 8
// so that the piece starts and ends on a 16-byte boundary (and of the rows its
// lane groups work on at a time, where that many fit).  A
// workgroup must have tens of KB on their way to keep HBM busy: with one row per
// lane group (BLOCK / G rows, 9 KB at N = 577) the kernel ran slower than the
// general one.
template <class T>
constexpr int flat_chunk_rows(int N, int lanes, int ldsb) {
  const int rpb = kFlatBlock / lanes < 8 ? 8 : kFlatBlock / lanes;  // rows per pass, and 8 | rows
  const int cap = ldsb / (int)sizeof(T) / N;
  return cap >= rpb ? cap / rpb * rpb : cap / 8 * 8;
}

// Copies the `nelem` elements at `src` (16-byte aligned) into LDS and back out:
// whole packs, all of a thread's loads requested before the first is written
// to LDS (a loop of load-then-write would wait for memory once per round), and
// the tail of the tensor's last piece element by element.
template <class T, int BLOCK, int U>  // U packs a thread: BLOCK * U packs = the LDS of one tensor
__device__ __forceinline__ void flat_stage_in(const T* __restrict__ src, T* buf, int nelem) {
  constexpr int E = elems_per_pack<T>::value;
  typedef typename Pack<T, E>::vec_t vec_t;
  const int nfull = nelem / E;
  Pack<T, E> p[U];
#pragma unroll
  for (int u = 0; u < U; ++u) {
    const int pk = (int)threadIdx.x + u * BLOCK;
    if (u * BLOCK < nfull)  // uniform
      p[u] = Pack<T, E>::load_stream(src + (pk < nfull ? pk : 0) * E);
  }
#pragma unroll
  for (int u = 0; u < U; ++u) {
    const int pk = (int)threadIdx.x + u * BLOCK;
    if (u * BLOCK < nfull && pk < nfull) *reinterpret_cast<vec_t*>(buf + pk * E) = p[u].v;
  }
  const int t = nfull * E + (int)threadIdx.x;
  if (t < nelem) buf[t] = src[t];
}
// The same for two tensors (the backward's grad and y): all loads of both before
// the first LDS write.
template <class T, int BLOCK, int U>
__device__ __forceinline__ void flat_stage_in2(const T* __restrict__ src0, T* buf0,
                                               const T* __restrict__ src1, T* buf1, int nelem) {
  constexpr int E = elems_per_pack<T>::value;
  typedef typename Pack<T, E>::vec_t vec_t;
  const int nfull = nelem / E;
  Pack<T, E> p[U], q[U];
#pragma unroll
  for (int u = 0; u < U; ++u) {
    const int pk = (int)threadIdx.x + u * BLOCK;
    if (u * BLOCK < nfull) {  // uniform
      p[u] = Pack<T, E>::load_stream(src0 + (pk < nfull ? pk : 0) * E);
      q[u] = Pack<T, E>::load_stream(src1 + (pk < nfull ? pk : 0) * E);
    }
  }
#pragma unroll
  for (int u = 0; u < U; ++u) {
    const int pk = (int)threadIdx.x + u * BLOCK;
    if (u * BLOCK < nfull && pk < nfull) {
      *reinterpret_cast<vec_t*>(buf0 + pk * E) = p[u].v;
      *reinterpret_cast<vec_t*>(buf1 + pk * E) = q[u].v;
    }
  }
  const int t = nfull * E + (int)threadIdx.x;
  if (t < nelem) {
    buf0[t] = src0[t];
    buf1[t] = src1[t];
  }
}
template <class T, int BLOCK, int U>
__device__ __forceinline__ void flat_stage_out(T* __restrict__ dst, const T* buf, int nelem) {
  constexpr int E = elems_per_pack<T>::value;
  typedef typename Pack<T, E>::vec_t vec_t;
  const int nfull = nelem / E;
#pragma unroll
  for (int u = 0; u < U; ++u) {
    const int pk = (int)threadIdx.x + u * BLOCK;
    if (u * BLOCK < nfull && pk < nfull) {
      Pack<T, E> p;
      p.v = *reinterpret_cast<const vec_t*>(buf + pk * E);
      p.store_stream(dst + pk * E);
    }
  }
  const int t = nfull * E + (int)threadIdx.x;
  if (t < nelem) dst[t] = buf[t];
}

// A lane's pack c of a row held in LDS: elements (c * G + lane) * E ... + E of the
// row, read with one LDS access at the row's own (element) alignment.  Reads may
// run past the row end into the next row or the padding of the buffer; `nv` is
// the number of elements that belong to the row.
template <class T, int E>
__device__ __forceinline__ Pack<T, E> flat_row_pack(const T* rowb, int j) {
  return Pack<T, E>::load(rowb + j);
}
template <class T, int E>
__device__ __forceinline__ void flat_row_store(T* rowb, int j, int nv, const Pack<T, E>& p) {
  if (nv >= E) {
    p.store(rowb + j);
  } else {
#pragma unroll
    for (int i = 0; i < E; ++i)
      if (i < nv) rowb[j + i] = p.v[i];
  }
}

// Short ragged rows through LDS (softmax_fwd_flat_kernel / softmax_bwd_flat_kernel).
constexpr int kFlatWholePackRowsMaxPacks = 12;
struct FlatLayout {
  int g = 0;   // lanes per row (0: the call does not qualify)
  int vp = 0;  // packs per lane
};

// The (lanes 1..64, packs per lane 1..4) with the fewest idle pack slots; among
// equals the one nearest two packs a lane, the layout the resident kernels prefer.
// Measured against "two packs a lane on the fewest lanes that hold the row",
// interleaved, bf16 forward / backward in us: rows of 13: 19.5 / 18.5 -> 10.6 / 8.6,
// 21: 30.0 / 25.9 -> 14.1 / 16.1, 45: 20.3 / 22.8 -> 16.5 / 20.6, 577 (73 packs: 32 x 3
// instead of 64 x 2): 72.1 / 96.5 -> 67.8 / 96.3, 750: 54.0 / 76.2 -> 51.2 / 75.1; 93
// and 129 lose 5-10 % in the backward (13.1 -> 14.6, 33.1 -> 34.8).
template <class T>
inline FlatLayout flat_layout(const Plan& plan, int64_t M, int N, const void* p0, const void* p1,
                              const void* p2) {
  constexpr int E = elems_per_pack<T>::value;
  FlatLayout f;
  if (plan.forced || M < 1 || N > 64 * kFlatMaxPacks * E) return f;
  if ((((uintptr_t)p0) | ((uintptr_t)p1) | ((uintptr_t)p2)) & 15) return f;
  const int packs = (N + E - 1) / E;
  // rows of whole packs qualify only when they are very short (see below)
  if (plan.fast && (packs > kFlatWholePackRowsMaxPacks || !plan.resident)) return f;
  int best_slots = 0, best_rank = 0;
  for (int g = 1; g <= 64; g <<= 1) {
    const int vp = (packs + g - 1) / g;
    if (vp > kFlatMaxPacks) continue;
    // (one or two lanes a row: rows of 1, 2 and 4 packs, which fill them exactly; 3 packs on
    // 2 x 2 measured 5-10 % behind 4 x 1 in the forward)
    if (g < 4 && (vp > 2 || g * vp != packs)) continue;
    const int slots = g * vp;
    const int rank = vp == 2 ? 0 : (vp == 3 ? 1 : (vp == 1 ? 2 : 3));
    if (f.g == 0 || slots < best_slots || (slots == best_slots && rank < best_rank)) {
      f.g = g;
      f.vp = vp;
      best_slots = slots;
      best_rank = rank;
    }
  }
  // Rows of whole packs: only up to 12 packs and where the resident layout leaves a
  // quarter of its pack slots idle, e.g. 9 or 10 packs on 8 lanes x 2 (bf16 rows of 72:
  // 36.6 / 52.5 -> 31.2 / 44.3 us, of 80: 40.9 / 57.6 -> 33.2 / 48.2 us, of 24: 32.1 / 29.4
  // -> 18.1 / 25.1 us); from 17 packs on it measured the same or slower (520: +2 %, 1032:
  // the backward +30 %).
  if (plan.fast && best_slots * 4 > plan.G * plan.V * 3) f = FlatLayout{};
  return f;
}

// One case per (lanes, packs per lane) of a launch switch keyed by lanes * 8 + packs.
#define ROWNORM_FLAT_CASES(CASE, GL) CASE(GL, 1) CASE(GL, 2) CASE(GL, 3) CASE(GL, 4)
#define ROWNORM_FLAT_CASES_NARROW(CASE, GL) CASE(GL, 1) CASE(GL, 2)
#define ROWNORM_FLAT_ALL(CASE)                                                       \
  ROWNORM_FLAT_CASES_NARROW(CASE, 1) ROWNORM_FLAT_CASES_NARROW(CASE, 2) ROWNORM_FLAT_CASES(CASE, 4) \
  ROWNORM_FLAT_CASES(CASE, 8) ROWNORM_FLAT_CASES(CASE, 16) ROWNORM_FLAT_CASES(CASE, 32) \
  ROWNORM_FLAT_CASES(CASE, 64)

}  // namespace rownorm
