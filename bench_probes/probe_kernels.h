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

// The read-only counterpart: the same walk, the data XOR-folded instead of stored (*sink is written only if the fold
// equals a constant, which it does not). Whether rows matter to a read stream at all.
__global__ __launch_bounds__(256) void stream_probe_flat_read_kernel(const u32x4* __restrict__ src, int64_t nvec,
                                                                     uint32_t magic, uint32_t* sink) {
  constexpr int U = 8;
  const int64_t stride = static_cast<int64_t>(gridDim.x) * 256 * U;
  int64_t base = (static_cast<int64_t>(blockIdx.x) * 256 + (threadIdx.x >> 6) * 64) * U + (threadIdx.x & 63);
  uint32_t fold = 0;
  for (; base + (U - 1) * 64 < nvec; base += stride) {
    u32x4 v[U];
#pragma unroll
    for (int u = 0; u < U; ++u) v[u] = __builtin_nontemporal_load(src + base + u * 64);
#pragma unroll
    for (int u = 0; u < U; ++u) fold ^= v[u].x ^ v[u].y ^ v[u].z ^ v[u].w;
  }
  for (int u = 0; u < U; ++u) {
    const int64_t k = base + u * 64;
    if (k < nvec) {
      const u32x4 v = __builtin_nontemporal_load(src + k);
      fold ^= v.x ^ v.y ^ v.z ^ v.w;
    }
  }
  if (fold == magic) *sink = fold;
}

// Matrix-core probe: what the part sustains on bf16 matrix instructions with nothing else in the way. 512 threads per
// workgroup (two wavefronts per SIMD, like the LM-head kernels), every wavefront issues `iters` rounds of the products
// of a 64 x 128 wavefront tile over 16 contraction elements on register operands. `random_operands` fills the
// fragments with pseudo-random bf16 values in (-1, 1) (what real activations and weights look like to the multipliers);
// otherwise every element is a small integer multiple of 1/8, the same in all products. The part is power-managed: the
// clock it holds, and with it the rate, depends on how much the operand bits toggle. Thread 0 of workgroup 0 reports how
// many shader clocks and how many ticks of the constant-rate wall clock its loop took, i.e. the clock the part ran at.
typedef __bf16 probe_bf16x8 __attribute__((ext_vector_type(8)));
typedef float probe_f32x16 __attribute__((ext_vector_type(16)));

__device__ __forceinline__ float probe_uniform(uint32_t x) {   // (-1, 1), from a 32-bit mix
  x ^= x >> 16;
  x *= 0x7feb352dU;
  x ^= x >> 15;
  x *= 0x846ca68bU;
  x ^= x >> 16;
  return static_cast<float>(static_cast<int32_t>(x)) * (1.0f / 2147483648.0f);
}

typedef float probe_f32x4 __attribute__((ext_vector_type(4)));

// SHAPE 32: v_mfma_f32_32x32x16_bf16, 2 x 4 blocks per round; SHAPE 16: v_mfma_f32_16x16x32_bf16, 4 x 8 blocks per round
// (the instruction of the LM-head kernels). `iters` counts 64 x 128 x 16 wavefront tiles (2 * 64 * 128 * 16 flops); a
// SHAPE 16 round covers 32 contraction elements, so it runs iters / 2 rounds.
template <int SHAPE>
__global__ __launch_bounds__(512, 1) void mfma_probe_kernel(int64_t iters, int random_operands, float* __restrict__ sink,
                                                            int64_t* __restrict__ clocks) {
  constexpr int NA = SHAPE == 32 ? 2 : 4, NB = SHAPE == 32 ? 4 : 8;
  probe_bf16x8 a[NA], b[NB];
  const uint32_t me = blockIdx.x * 512u + threadIdx.x;
#pragma unroll
  for (int f = 0; f < NA + NB; ++f)
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const float v = random_operands ? probe_uniform(me * 96u + f * 8u + i) : 0.125f * static_cast<float>((threadIdx.x + i) & 7);
      if (f < NA) a[f][i] = static_cast<__bf16>(v); else b[f - NA][i] = static_cast<__bf16>(v);
    }
  float total = 0.f;
  long long c0, w0;
  if constexpr (SHAPE == 32) {
    probe_f32x16 acc[2][4];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;
    c0 = clock64();
    w0 = wall_clock64();
    for (int64_t it = 0; it < iters; ++it) {
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[i], b[j], acc[i][j], 0, 0, 0);
    }
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int v = 0; v < 16; ++v) total += acc[i][j][v];
  } else {
    probe_f32x4 acc[4][8];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 8; ++j)
#pragma unroll
        for (int v = 0; v < 4; ++v) acc[i][j][v] = 0.f;
    c0 = clock64();
    w0 = wall_clock64();
    for (int64_t it = 0; it < iters / 2; ++it) {
#pragma unroll
      for (int j = 0; j < 8; ++j)
#pragma unroll
        for (int i = 0; i < 4; ++i) acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[i], b[j], acc[i][j], 0, 0, 0);
    }
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 8; ++j)
#pragma unroll
        for (int v = 0; v < 4; ++v) total += acc[i][j][v];
  }
  if (clocks != nullptr && blockIdx.x == 0 && threadIdx.x == 0) {
    clocks[0] = clock64() - c0;
    clocks[1] = wall_clock64() - w0;
  }
  if (total == 12345.678f) sink[0] = total;   // keeps the products alive; practically never true
}

}  // namespace vrl
