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

// Optimization barrier on a register-resident pack of 16-bit elements.  A row
// that must survive a cross-lane reduction is kept in storage format (two
// elements per VGPR) and widened to fp32 again in each pass over it; without
// the barrier the compiler would keep the widened copy alive across the
// reduction instead, doubling the registers the row occupies.
template <class T, int E>
__device__ __forceinline__ void keep_packed(Pack<T, E>& p) {
  if constexpr (sizeof(T) == 2 && E == 8) {
    typedef uint32_t raw_t __attribute__((ext_vector_type(4)));
    raw_t r = __builtin_bit_cast(raw_t, p.v);
    asm volatile("" : "+v"(r));
    p.v = __builtin_bit_cast(typename Pack<T, E>::vec_t, r);
  }
}

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

// Row accessors used by the register-resident kernels.
//
// FAST (the row length is a whole number of packs): the load is unconditional
// -- a lane whose pack lies beyond the row reads the row's first pack instead
// and the value is replaced by `fill` with a select -- so the V loads of a lane
// are straight-line code that the hardware issues back to back.  `row` must
// point at a readable row even when `ok` is false (callers clamp the index).
// Otherwise: the general loader above (handles a pack that straddles the row
// end element by element, at the price of a branch per pack).
template <class T, int E, bool STREAM, bool FAST>
__device__ __forceinline__ Pack<T, E> row_load(const T* row, int e0, int n, bool ok, float fill) {
  if constexpr (FAST) {
    const bool inb = e0 < n;
    const T* p = row + (inb ? e0 : 0);
    Pack<T, E> r = STREAM ? Pack<T, E>::load_stream(p) : Pack<T, E>::load(p);
    const Pack<T, E> f = Pack<T, E>::splat(fill);
    if (!(inb && ok)) r = f;
    return r;
  } else {
    return load_row_pack<T, E, STREAM>(row, e0, n, ok, fill);
  }
}

template <class T, int E, bool STREAM, bool FAST>
__device__ __forceinline__ void row_store(T* row, int e0, int n, bool ok, const Pack<T, E>& p) {
  if constexpr (FAST) {
    if (ok && e0 < n) {
      if (STREAM)
        p.store_stream(row + e0);
      else
        p.store(row + e0);
    }
  } else {
    store_row_pack<T, E, STREAM>(row, e0, n, ok, p);
  }
}

}  // namespace rownorm
