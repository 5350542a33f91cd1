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
#include <type_traits>
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace rownorm {

using f16 = _Float16;
using bf16 = __bf16;

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
    r.v = __builtin_nontemporal_load(reinterpret_cast<const uvec_t*>(p));
    return r;
  }
  __device__ __forceinline__ static Pack load(const T* p) {
    Pack r;
    r.v = *reinterpret_cast<const uvec_t*>(p);
    return r;
  }
  __device__ __forceinline__ void store_stream(T* p) const {
    __builtin_nontemporal_store(v, reinterpret_cast<uvec_t*>(p));
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

// Loads from wavefront-uniform addresses of memory that no kernel writes while
// it runs (inputs, weights, saved statistics).  Through the constant address
// space the compiler issues them on the scalar unit, where they neither take a
// vector register nor count among the vector memory operations a row loop waits
// for; a plain load from a uniform address becomes a vector load as soon as a
// barrier precedes it, because the barrier's fence may have changed any memory.
template <class U>
__device__ __forceinline__ U uniform_load(const void* p) {
  return *(const __attribute__((address_space(4))) U*)(uintptr_t)p;
}

// Element i (wavefront-uniform) of an array of 16- or 32-bit values: the aligned
// 32-bit word that holds it is loaded -- the scalar unit has no 16-bit loads --
// and value() picks the element out of it.  The word lies within the 4 bytes
// around the element, so nothing beyond the array's last word is touched.
template <class WT>
struct UniformElem {
  uint32_t word;
  uint32_t shift;
  __device__ __forceinline__ static UniformElem load(const WT* w, int64_t i) {
    const char* p = reinterpret_cast<const char*>(w + i);
    UniformElem r;
    r.shift = 0;
    if constexpr (sizeof(WT) == 2) {
      const uint32_t odd = (uint32_t)(reinterpret_cast<uintptr_t>(p) & 2);
      p -= odd;
      r.shift = odd * 8u;
    }
    r.word = uniform_load<uint32_t>(p);
    return r;
  }
  __device__ __forceinline__ float value() const {
    if constexpr (sizeof(WT) == 4) {
      return __builtin_bit_cast(float, word);
    } else {
      return (float)__builtin_bit_cast(WT, (uint16_t)(word >> shift));
    }
  }
};

// The lane index as a value the compiler cannot trace back to threadIdx, and
// that exists only once `after` does: the pack offsets derived from it are then
// computed where they are used (after a reduction, say) instead of ahead of the
// row loop, where each would hold a register for the whole kernel.
template <bool ON = true>
__device__ __forceinline__ int lane_after(int lane, float& after) {
  if constexpr (ON) asm volatile("" : "+v"(lane), "+v"(after));
  return lane;
}

// The same at the top of a row loop, with nothing to wait for.
template <bool ON = true>
__device__ __forceinline__ int lane_again(int lane) {
  if constexpr (ON) asm volatile("" : "+v"(lane));
  return lane;
}

// Loads the pack that starts at element `e0` of a row whose elements are
// [lo, n) of `row`.  A pack that lies wholly inside the row is one 128-bit load;
// a pack that straddles either end of the row is read element by element and
// padded with `fill`; a pack wholly outside the row is all `fill`.  Nothing
// outside [lo, n) is touched.  The element loads go to clamped addresses, all
// valid, so they are independent of one another and of the padding: E requests
// in flight and one wait, not a load-and-wait per element.
template <class T, int E, bool STREAM>
__device__ __forceinline__ Pack<T, E> load_row_pack(const T* row, int e0, int n, bool row_ok,
                                                    float fill, int lo = 0) {
  if (row_ok && e0 >= lo && e0 + E <= n) {
    return STREAM ? Pack<T, E>::load_stream(row + e0) : Pack<T, E>::load(row + e0);
  }
  Pack<T, E> r = Pack<T, E>::splat(fill);
  if (row_ok && e0 < n && e0 + E > lo) {
    // the index arithmetic of this rare path stays inside it: computed ahead of
    // the row loop it would hold registers in every lane for the whole kernel
    asm volatile("" : "+v"(e0));
    T t[E];
#pragma unroll
    for (int i = 0; i < E; ++i) {
      int j = e0 + i;
      j = j < lo ? lo : j;
      j = j >= n ? n - 1 : j;
      t[i] = row[j];
    }
#pragma unroll
    for (int i = 0; i < E; ++i)
      if (e0 + i >= lo && e0 + i < n) r.v[i] = t[i];
  }
  return r;
}

// The same for a row seen through a window whose packs are 16-byte aligned
// (see window_head below), in two steps.  A pack that holds any element of the
// row lies in that element's page, so it is read whole: one unconditional
// 128-bit load, like the fast kernels', and a lane's loads are straight-line
// code.  trim_window_pack then replaces the elements outside [lo, n) by `fill`;
// callers run it over their packs after all of them have been requested.
// `win` must be the window of a readable row even when `ok` is false (callers
// clamp the row index); lo < E.
template <class T, int E, bool STREAM>
__device__ __forceinline__ Pack<T, E> load_window_pack(const T* win, int e0, int n, bool ok,
                                                       float fill) {
  const bool inb = ok && e0 < n;
  const T* p = win + (inb ? e0 : 0);
  Pack<T, E> r = STREAM ? Pack<T, E>::load_stream(p) : Pack<T, E>::load(p);
  const Pack<T, E> f = Pack<T, E>::splat(fill);
  if (!inb) r = f;
  return r;
}

// LOCAL keeps the index arithmetic inside the branch, as load_row_pack does: the
// softmax backward, which holds two tensors' packs, gains registers by it (16-bit
// ragged rows on two packs a lane 70-74 -> 56-60 VGPRs: eight wavefronts a SIMD);
// the forward fits 64 registers either way and measured 0-10 % slower with it.
template <class T, int E, bool LOCAL = false>
__device__ __forceinline__ void trim_window_pack(Pack<T, E>& r, int e0, int n, float fill,
                                                 int lo) {
  if (e0 < n && (e0 < lo || e0 + E > n)) {
    if constexpr (LOCAL) asm volatile("" : "+v"(e0));
#pragma unroll
    for (int i = 0; i < E; ++i)
      if (e0 + i < lo || e0 + i >= n) r.v[i] = (T)fill;
  }
}

template <class T, int E, bool STREAM>
__device__ __forceinline__ void store_row_pack(T* row, int e0, int n, bool row_ok,
                                               const Pack<T, E>& p, int lo = 0) {
  if (!row_ok) return;
  if (e0 >= lo && e0 + E <= n) {
    if (STREAM)
      p.store_stream(row + e0);
    else
      p.store(row + e0);
  } else if (e0 < n && e0 + E > lo) {
    asm volatile("" : "+v"(e0));  // as in load_row_pack
#pragma unroll
    for (int i = 0; i < E; ++i)
      if (e0 + i >= lo && e0 + i < n) row[e0 + i] = p.v[i];
  }
}

// The packs p0 + t, p0 + t + BLOCK, ... below p1 of thread t, U at a time: the
// loads of U packs are issued (`fetch`) before the first of them is used (`use`),
// so a lane keeps U requests in flight instead of one.  Packs below `pfull` =
// N / E lie wholly inside the row: for them the callbacks get std::true_type and
// move plain 128-bit packs, straight-line code that the compiler can keep in
// flight; a branch around a load (the ragged path of load_row_pack) stops that,
// so only the last, ragged pack of a row (std::false_type) takes that path.
//   fetch(pk, whole) -> data        use(pk, data, whole)
template <int U, int BLOCK, class Fetch, class Use>
__device__ __forceinline__ void for_packs(int64_t p0, int64_t p1, int64_t pfull, Fetch fetch,
                                          Use use) {
  const int64_t pe = p1 < pfull ? p1 : pfull;
  int64_t pk = p0 + threadIdx.x;
  using Data = decltype(fetch(pk, std::true_type{}));
  for (; pk + (int64_t)(U - 1) * BLOCK < pe; pk += (int64_t)U * BLOCK) {
    Data d[U];
#pragma unroll
    for (int u = 0; u < U; ++u) d[u] = fetch(pk + (int64_t)u * BLOCK, std::true_type{});
#pragma unroll
    for (int u = 0; u < U; ++u) use(pk + (int64_t)u * BLOCK, d[u], std::true_type{});
  }
  for (; pk < pe; pk += BLOCK) use(pk, fetch(pk, std::true_type{}), std::true_type{});
  for (; pk < p1; pk += BLOCK) use(pk, fetch(pk, std::false_type{}), std::false_type{});
}

// One pack of a row of n elements at element e0: a plain 128-bit access when the
// caller knows it lies inside the row (WHOLE), load_row_pack / store_row_pack otherwise.
template <class T, int E, bool STREAM, bool WHOLE>
__device__ __forceinline__ Pack<T, E> load_pack_of(const T* row, int64_t e0, int n, float fill) {
  if constexpr (WHOLE)
    return STREAM ? Pack<T, E>::load_stream(row + e0) : Pack<T, E>::load(row + e0);
  else
    return load_row_pack<T, E, STREAM>(row, (int)e0, n, true, fill);
}

template <class T, int E, bool STREAM, bool WHOLE>
__device__ __forceinline__ void store_pack_of(T* row, int64_t e0, int n, const Pack<T, E>& p) {
  if constexpr (WHOLE) {
    if (STREAM)
      p.store_stream(row + e0);
    else
      p.store(row + e0);
  } else {
    store_row_pack<T, E, STREAM>(row, (int)e0, n, true, p);
  }
}

// Ragged rows (a row length that is not a whole number of packs puts every row
// at a different 2- or 4-byte alignment) are addressed through a window that
// starts on a 16-byte boundary of `row`'s memory: the row's first element sits
// `window_head(row)` elements into it.  Every whole pack of the window is then an
// aligned 128-bit access (a 128-bit access at a 2-byte alignment costs about
// twice as much), and only the window's first and last pack are moved element
// by element.  Tensors that share the row index keep a constant alignment
// relative to the window (the same one, when their base addresses are congruent
// modulo 16 bytes).
template <class T, int E>
__device__ __forceinline__ int window_head(const T* row) {
  return (int)((reinterpret_cast<uintptr_t>(row) / sizeof(T)) % (unsigned)E);
}

// Whether the packs of tensor `b` are 16-byte aligned in a window laid over the
// same rows of tensor `a` (same element type, same row length).
template <class T>
__device__ __forceinline__ bool same_pack_alignment(const T* a, const T* b) {
  return ((reinterpret_cast<uintptr_t>(a) ^ reinterpret_cast<uintptr_t>(b)) & 15u) == 0;
}

// Row accessors used by the register-resident kernels.
//
// FAST (the row length is a whole number of packs): the load is unconditional
// -- a lane whose pack lies beyond the row reads the row's first pack instead
// and the value is replaced by `fill` with a select -- so the V loads of a lane
// are straight-line code that the hardware issues back to back.  `row` must
// point at a readable row even when `ok` is false (callers clamp the index).
// Otherwise: the general loaders above -- `whole` (the row is seen through a
// window of 16-byte aligned packs) picks the one that reads boundary packs in
// full and leaves the trimming to the caller (row_trim), else a pack that
// straddles an end of the row [lo, n) is read element by element, at the price
// of a branch per pack.
template <class T, int E, bool STREAM, bool FAST>
__device__ __forceinline__ Pack<T, E> row_load(const T* row, int e0, int n, bool ok, float fill,
                                               int lo = 0, bool whole = false) {
  if constexpr (FAST) {
    const bool inb = e0 < n;
    const T* p = row + (inb ? e0 : 0);
    Pack<T, E> r = STREAM ? Pack<T, E>::load_stream(p) : Pack<T, E>::load(p);
    const Pack<T, E> f = Pack<T, E>::splat(fill);
    if (!(inb && ok)) r = f;
    return r;
  } else {
    if (whole) return load_window_pack<T, E, STREAM>(row, e0, n, ok, fill);
    return load_row_pack<T, E, STREAM>(row, e0, n, ok, fill, lo);
  }
}

// After row_load(..., whole): `fill` for the elements of the pack outside [lo, n).
template <class T, int E, bool FAST, bool LOCAL = false>
__device__ __forceinline__ void row_trim(Pack<T, E>& r, int e0, int n, float fill, int lo,
                                         bool whole) {
  if constexpr (!FAST) {
    if (whole) trim_window_pack<T, E, LOCAL>(r, e0, n, fill, lo);
  }
}

template <class T, int E, bool STREAM, bool FAST>
__device__ __forceinline__ void row_store(T* row, int e0, int n, bool ok, const Pack<T, E>& p,
                                          int lo = 0) {
  if constexpr (FAST) {
    if (ok && e0 < n) {
      if (STREAM)
        p.store_stream(row + e0);
      else
        p.store(row + e0);
    }
  } else {
    store_row_pack<T, E, STREAM>(row, e0, n, ok, p, lo);
  }
}

}  // namespace rownorm
