// 16-byte register packs of row elements and their fp32 views (gfx950, wave64).
//
// A Pack<T> is the unit every lane moves between HBM and registers: 16 bytes,
// i.e. 4 fp32 or 8 fp16/bf16 elements, read with one global_load_dwordx4 and
// written with one global_store_dwordx4.  Pointers handed to the library carry
// no alignment promise, so the pack pointer types are declared with the element
// alignment only; gfx950 runs with unaligned global access enabled and the
// compiler still emits the single 128-bit instruction.
//
// Role in the reference: aligned_vector<T, n> (src/ATen/native/xpu/sycl/
// MemoryAccessUtils.h:232) and the can_vectorize_up_to ladder (MemoryAccess.h:
// 290-314), which drops to narrower accesses when a pointer is misaligned.
// Here the access stays 128-bit wide for every pointer and only a row tail
// shorter than one pack is moved element by element.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace rownorm {

using f16 = _Float16;
using bf16 = __bf16;

#ifndef ROWNORM_NT_LOAD
#define ROWNORM_NT_LOAD 1
#endif
#ifndef ROWNORM_NT_STORE
#define ROWNORM_NT_STORE 1
#endif

template <class T>
struct elems_per_pack {
  static constexpr int value = 16 / sizeof(T);
};

// E consecutive elements of T held in registers in storage format.
template <class T, int E>
struct Pack {
  typedef T vec_t __attribute__((ext_vector_type(E)));
  typedef vec_t uvec_t __attribute__((aligned(sizeof(T))));  // element-aligned view
  vec_t v;

  __device__ __forceinline__ static Pack zero() {
    Pack r;
#pragma unroll
    for (int i = 0; i < E; ++i) r.v[i] = (T)0.0f;
    return r;
  }
  __device__ __forceinline__ static Pack splat(float f) {
    Pack r;
#pragma unroll
    for (int i = 0; i < E; ++i) r.v[i] = (T)f;
    return r;
  }
  // Streaming (read-once / write-once) accesses carry the non-temporal hint.
  __device__ __forceinline__ static Pack load_stream(const T* p) {
    Pack r;
#if ROWNORM_NT_LOAD
    r.v = __builtin_nontemporal_load(reinterpret_cast<const uvec_t*>(p));
#else
    r.v = *reinterpret_cast<const uvec_t*>(p);
#endif
    return r;
  }
  __device__ __forceinline__ static Pack load(const T* p) {
    Pack r;
    r.v = *reinterpret_cast<const uvec_t*>(p);
    return r;
  }
  __device__ __forceinline__ void store_stream(T* p) const {
#if ROWNORM_NT_STORE
    __builtin_nontemporal_store(v, reinterpret_cast<uvec_t*>(p));
#else
    *reinterpret_cast<uvec_t*>(p) = v;
#endif
  }
  __device__ __forceinline__ void store(T* p) const { *reinterpret_cast<uvec_t*>(p) = v; }

  __device__ __forceinline__ float get(int i) const { return (float)v[i]; }
  __device__ __forceinline__ void set(int i, float f) { v[i] = (T)f; }
};

// Loads the pack that starts at element `e0` of a row of `n` elements.  A pack
// that lies wholly inside the row is one 128-bit load; the (at most one) pack
// that straddles the end of the row is read element by element and padded with
// `fill`; a pack wholly outside the row is all `fill`.
template <class T, int E, bool STREAM>
__device__ __forceinline__ Pack<T, E> load_row_pack(const T* row, int e0, int n, bool row_ok,
                                                    float fill) {
  if (row_ok && e0 + E <= n) {
    return STREAM ? Pack<T, E>::load_stream(row + e0) : Pack<T, E>::load(row + e0);
  }
  Pack<T, E> r = Pack<T, E>::splat(fill);
  if (row_ok && e0 < n) {
#pragma unroll
    for (int i = 0; i < E; ++i)
      if (e0 + i < n) r.v[i] = row[e0 + i];
  }
  return r;
}

template <class T, int E, bool STREAM>
__device__ __forceinline__ void store_row_pack(T* row, int e0, int n, bool row_ok,
                                               const Pack<T, E>& p) {
  if (!row_ok) return;
  if (e0 + E <= n) {
    if (STREAM)
      p.store_stream(row + e0);
    else
      p.store(row + e0);
  } else if (e0 < n) {
#pragma unroll
    for (int i = 0; i < E; ++i)
      if (e0 + i < n) row[e0 + i] = p.v[i];
  }
}

}  // namespace rownorm
