// Measurement aid, no decoding: the memory side of the decode kernels alone.
//
// ep_hip_probe_store_pattern writes `vectors` 16-byte vectors exactly as a bf16 lattice decode of tiles of `tile_vectors`
// vectors does: one tile per 32-lane half of a persistent grid of 16-wave workgroups (two per CU), every half its tile
// top-down in groups of 32 consecutive vectors, 16 bytes per lane and store instruction. What this takes is what the
// decode kernels' own output costs whatever feeds it; bench.py --workload store_pattern reports it beside a plain fill.
#include <hip/hip_runtime.h>

#include "entropack_hip.h"
#include "ep_common.hpp"

namespace ep {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

template <int POLICY>     // 0: streaming stores (the decode kernels'), 1: stores through the cache, 2: streaming, heads delayed
__global__ __launch_bounds__(1024) void store_pattern_kernel(uint8_t* __restrict__ out, int64_t vectors, int tile_vectors) {
  const int lane = threadIdx.x & 63, half = lane >> 5, l32 = lane & 31;
  const int64_t wave = static_cast<int64_t>(blockIdx.x) * (blockDim.x >> 6) + (threadIdx.x >> 6);
  const int64_t waves = static_cast<int64_t>(gridDim.x) * (blockDim.x >> 6);
  const int64_t tiles = (vectors + tile_vectors - 1) / tile_vectors;
  for (int64_t pair = wave; 2 * pair < tiles; pair += waves) {
    const int64_t tile = 2 * pair + half;
    if (tile >= tiles) continue;
    const int64_t first = tile * tile_vectors;
    const int64_t left = vectors - first;
    const int count = static_cast<int>(left < tile_vectors ? left : tile_vectors);
    if (POLICY == 2) {
      // The first `late` lanes of a group hold the vectors in front of the next 64-byte boundary: they wait one turn and go
      // out with the group below, so that every store instruction covers whole 64-byte lines.
      const int late = static_cast<int>((4 - (first & 3)) & 3);
      for (int offset = (count - 1) & ~31; offset >= -32; offset -= 32) {
        const int vector = l32 < late ? offset + 32 + l32 : offset + l32;
        if (vector < 0 || vector >= count || (offset < 0 && l32 >= late)) continue;
        const u32x4 value = {static_cast<uint32_t>(tile), static_cast<uint32_t>(vector & ~31), static_cast<uint32_t>(l32), 0u};
        __builtin_nontemporal_store(value, reinterpret_cast<u32x4*>(out + 16 * (first + vector)));
      }
      continue;
    }
    for (int offset = (count - 1) & ~31; offset >= 0; offset -= 32) {
      if (offset + l32 >= count) continue;
      const u32x4 value = {static_cast<uint32_t>(tile), static_cast<uint32_t>(offset), static_cast<uint32_t>(l32), 0u};
      u32x4* to = reinterpret_cast<u32x4*>(out + 16 * (first + offset + l32));
      if (POLICY == 0) __builtin_nontemporal_store(value, to);
      else *to = value;
    }
  }
}

}  // namespace ep

extern "C" int ep_hip_probe_store_pattern(void* out_dev, int64_t vectors, int tile_vectors, int through_cache, void* stream) {
  if (out_dev == nullptr || vectors <= 0 || tile_vectors <= 0 || reinterpret_cast<uintptr_t>(out_dev) % 16 != 0) return EP_HIP_EINVAL;
  int device = 0, cus = 0;
  EP_HIP_TRY(hipGetDevice(&device));
  EP_HIP_TRY(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, device));
  const dim3 grid(static_cast<unsigned>(2 * (cus > 0 ? cus : 256))), block(1024);
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (through_cache == 2) hipLaunchKernelGGL(ep::store_pattern_kernel<2>, grid, block, 0, s, static_cast<uint8_t*>(out_dev), vectors, tile_vectors);
  else if (through_cache) hipLaunchKernelGGL(ep::store_pattern_kernel<1>, grid, block, 0, s, static_cast<uint8_t*>(out_dev), vectors, tile_vectors);
  else hipLaunchKernelGGL(ep::store_pattern_kernel<0>, grid, block, 0, s, static_cast<uint8_t*>(out_dev), vectors, tile_vectors);
  EP_HIP_TRY(hipGetLastError());
  return EP_HIP_OK;
}
