// Memory-system probes: what the part delivers for the row kernels' access pattern with no arithmetic in the way.
// They are the ceilings the row kernels are measured against (a plain read for the forward kernel, a plain copy for
// the backward kernel), not part of the scoring path.
//
// A workgroup of WAVES wavefronts owns one contiguous "row" of `vecs_per_row` 16-byte vectors; wave w reads the
// w-th contiguous U KiB slice of every WAVES*U KiB block with non-temporal 128-bit loads, exactly like
// block_reduce_range. READ folds the data into one word per lane (XOR) and stores it only if it equals a value the
// caller chose never to occur; COPY stores every vector to the same position of `dst` with non-temporal stores.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "rowscore_kernels.h"

namespace vrl {

template <int WAVES, int U, bool COPY>
__global__ __launch_bounds__(WAVES * 64) void stream_probe_kernel(const u32x4* __restrict__ src,
                                                                  u32x4* __restrict__ dst, int64_t vecs_per_row,
                                                                  uint32_t never, uint32_t* __restrict__ sink) {
  constexpr int NTHR = WAVES * 64;
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const u32x4* vp = src + static_cast<int64_t>(blockIdx.x) * vecs_per_row;
  u32x4* dp = dst + static_cast<int64_t>(blockIdx.x) * vecs_per_row;
  uint32_t acc = 0;
  constexpr int64_t kBatchVecs = static_cast<int64_t>(NTHR) * U;
  const int64_t nfull = vecs_per_row / kBatchVecs;
  for (int64_t j = 0; j < nfull; ++j) {
    const int64_t base = (j * WAVES + wave) * (U * 64) + lane;
    u32x4 v[U];
#pragma unroll
    for (int u = 0; u < U; ++u) v[u] = __builtin_nontemporal_load(vp + base + u * 64);
#pragma unroll
    for (int u = 0; u < U; ++u) {
      if constexpr (COPY) {
        __builtin_nontemporal_store(v[u], dp + base + u * 64);
      } else {
        acc ^= v[u].x ^ v[u].y ^ v[u].z ^ v[u].w;
      }
    }
  }
  for (int64_t k = nfull * kBatchVecs + tid; k < vecs_per_row; k += NTHR) {
    const u32x4 v = __builtin_nontemporal_load(vp + k);
    if constexpr (COPY) {
      __builtin_nontemporal_store(v, dp + k);
    } else {
      acc ^= v.x ^ v.y ^ v.z ^ v.w;
    }
  }
  if constexpr (!COPY) {
    if (acc == never) sink[0] = acc;
  }
}

// The same copy without rows: a fixed number of workgroups of 4 wavefronts walk the whole buffer, each wavefront moving
// 8 KiB (8 non-temporal 128-bit loads per lane, then 8 stores) per trip. The best of the shapes tried for a read+write
// stream on this part; it bounds what any row-shaped kernel that reads N bytes and writes N bytes can reach.
__global__ __launch_bounds__(256) void stream_probe_flat_copy_kernel(const u32x4* __restrict__ src, u32x4* __restrict__ dst,
                                                                     int64_t nvec) {
  constexpr int U = 8;
  const int64_t stride = static_cast<int64_t>(gridDim.x) * 256 * U;
  int64_t base = (static_cast<int64_t>(blockIdx.x) * 256 + (threadIdx.x >> 6) * 64) * U + (threadIdx.x & 63);
  for (; base + (U - 1) * 64 < nvec; base += stride) {
    u32x4 v[U];
#pragma unroll
    for (int u = 0; u < U; ++u) v[u] = __builtin_nontemporal_load(src + base + u * 64);
#pragma unroll
    for (int u = 0; u < U; ++u) __builtin_nontemporal_store(v[u], dst + base + u * 64);
  }
  // what is left of the last, partial trip of this wavefront's slot
  for (int u = 0; u < U; ++u) {
    const int64_t k = base + u * 64;
    if (k < nvec) __builtin_nontemporal_store(__builtin_nontemporal_load(src + k), dst + k);
  }
}

}  // namespace vrl
