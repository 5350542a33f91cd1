// Plain streaming kernels of known traffic: what this GPU's memory system gives a
// kernel that does nothing but move 16-byte packs, in the three read : write mixes
// of this operator family (1 : 1 like a forward, 2 : 1 like a backward, reads
// only).  The benchmark reports them beside the operators, so that an operator's
// fraction of the 8 TB/s peak can be read against the fraction a bare copy
// reaches on the same box; rocprofv3's FETCH_SIZE / WRITE_SIZE readings are
// scaled by the same kernels.  Not part of the operator path.
#include "../../../include/mi355x_rownorm.h"

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace {

typedef uint32_t u4 __attribute__((ext_vector_type(4)));

// MODE 0: c = a.  1: c = a + b (32-bit integer adds).  2: every workgroup sums its
// share of a and b and writes one pack per thread.  Loads and stores carry the
// non-temporal hint like the operators' (without it a copy runs 8 % slower here).
template <int MODE, int U, int BLOCK>
__global__ void __launch_bounds__(BLOCK)
stream_probe_kernel(const u4* __restrict__ a, const u4* __restrict__ b, u4* __restrict__ c,
                    int64_t npacks) {
  u4 acc = {0, 0, 0, 0};
  constexpr int64_t tile = (int64_t)BLOCK * U;
  const int64_t ntiles = (npacks + tile - 1) / tile;
  for (int64_t t = blockIdx.x; t < ntiles; t += gridDim.x) {
    const int64_t base = t * tile + threadIdx.x;
    u4 va[U], vb[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int64_t i = base + u * BLOCK;
      const bool in = i < npacks;
      va[u] = __builtin_nontemporal_load(a + (in ? i : 0));
      if (MODE != 0) vb[u] = __builtin_nontemporal_load(b + (in ? i : 0));
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int64_t i = base + u * BLOCK;
      u4 v = va[u];
      if (MODE != 0) v += vb[u];
      if (MODE == 2) {
        if (i < npacks) acc += v;
      } else if (i < npacks) {
        __builtin_nontemporal_store(v, c + i);
      }
    }
  }
  if (MODE == 2) c[(int64_t)blockIdx.x * BLOCK + threadIdx.x] = acc;
}

}  // namespace

extern "C" int mi355x_rownorm_stream_probe(const void* a, const void* b, void* c, size_t bytes,
                                           int mode, void* stream) {
  if (mode < 0 || mode > 2) return ROWNORM_ERR_SHAPE;
  if (bytes == 0) return 0;
  if (!a || !c || (mode != 0 && !b)) return ROWNORM_ERR_NULL;
  if (bytes % 16 != 0 || (((uintptr_t)a | (uintptr_t)b | (uintptr_t)c) & 15u) != 0)
    return ROWNORM_ERR_SHAPE;
  const int64_t npacks = (int64_t)(bytes / 16);
  hipStream_t s = (hipStream_t)stream;
  // measured best on MI355X at 128 MiB a tensor: one workgroup per tile of 1024 packs
  // for the copy and the add, a grid of 2048 workgroups walking the tensor for the read
  if (mode == 0) {
    const int64_t tiles = (npacks + 1023) / 1024;
    hipLaunchKernelGGL((stream_probe_kernel<0, 4, 256>), dim3((unsigned)tiles), dim3(256), 0, s,
                       (const u4*)a, (const u4*)b, (u4*)c, npacks);
  } else if (mode == 1) {
    const int64_t tiles = (npacks + 1023) / 1024;
    hipLaunchKernelGGL((stream_probe_kernel<1, 2, 512>), dim3((unsigned)tiles), dim3(512), 0, s,
                       (const u4*)a, (const u4*)b, (u4*)c, npacks);
  } else {
    int64_t grid = (npacks + 1023) / 1024;
    if (grid > 2048) grid = 2048;
    if ((size_t)grid * 256 * 16 > bytes) return ROWNORM_ERR_SHAPE;  // c holds grid * 256 packs
    hipLaunchKernelGGL((stream_probe_kernel<2, 4, 256>), dim3((unsigned)grid), dim3(256), 0, s,
                       (const u4*)a, (const u4*)b, (u4*)c, npacks);
  }
  return (int)hipGetLastError();
}
