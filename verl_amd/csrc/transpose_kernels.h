// Out-of-place transposition of a 2-D array of 2- or 4-byte elements:
//   dst[c * dst_stride + r] = src[r * src_stride + c],  r < rows, c < cols.
// Pure byte movement (no arithmetic), bound by HBM: each workgroup moves one
// TILE x TILE block through LDS so that both the reads and the writes are
// 16-byte vectors along the contiguous axis of their array (256 B per tile row).
// The LM-head weight and the hidden states are brought into the operand order
// the library GEMM runs fastest in (both operands contiguous along the
// contraction axis) with this kernel.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace vrl {

typedef uint32_t tr_u32x4 __attribute__((ext_vector_type(4)));

template <int ES>
struct TransposeShape;
template <>
struct TransposeShape<2> {
  static constexpr int kTile = 128;                 // elements per tile side: 256 B per tile row
  static constexpr int kPitch = kTile / 2 + 1;      // LDS row pitch in 32-bit words (odd: spreads banks)
};
template <>
struct TransposeShape<4> {
  static constexpr int kTile = 64;
  static constexpr int kPitch = kTile + 1;
};

// grid.x = tiles_r * tiles_c (column tiles fastest), block = 256.
// vec_ok: both base pointers and both row pitches are multiples of 16 bytes.
template <int ES>
__global__ __launch_bounds__(256) void transpose_kernel(const char* __restrict__ src, int64_t rows, int64_t cols,
                                                        int64_t src_stride, char* __restrict__ dst,
                                                        int64_t dst_stride, int64_t tiles_c, int vec_ok) {
  using S = TransposeShape<ES>;
  constexpr int TILE = S::kTile;
  constexpr int P = S::kPitch;
  constexpr int EPV = 16 / ES;        // elements per 16-byte vector
  constexpr int VPR = TILE / EPV;     // vectors per tile row
  constexpr int NV = TILE * VPR / 256;  // vectors per thread
  __shared__ uint32_t lds[TILE * P];

  const int tid = threadIdx.x;
  const int64_t tr = static_cast<int64_t>(blockIdx.x) / tiles_c;
  const int64_t tc = static_cast<int64_t>(blockIdx.x) - tr * tiles_c;
  const int64_t r0 = tr * TILE;
  const int64_t c0 = tc * TILE;
  const bool full = vec_ok && (r0 + TILE <= rows) && (c0 + TILE <= cols);

  if (full) {
    tr_u32x4 v[NV];
#pragma unroll
    for (int k = 0; k < NV; ++k) {
      const int i = tid + k * 256;
      const int row = i / VPR, vec = i % VPR;
      v[k] = __builtin_nontemporal_load(
          reinterpret_cast<const tr_u32x4*>(src + ((r0 + row) * src_stride + c0) * ES + vec * 16));
    }
#pragma unroll
    for (int k = 0; k < NV; ++k) {
      const int i = tid + k * 256;
      const int row = i / VPR, vec = i % VPR;
      uint32_t* p = lds + row * P + vec * 4;
      p[0] = v[k].x;
      p[1] = v[k].y;
      p[2] = v[k].z;
      p[3] = v[k].w;
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < NV; ++k) {
      const int i = tid + k * 256;
      const int c = i / VPR, rv = i % VPR;   // output row c of the tile, vector rv along it
      tr_u32x4 o;
      if constexpr (ES == 4) {
        o.x = lds[(rv * 4 + 0) * P + c];
        o.y = lds[(rv * 4 + 1) * P + c];
        o.z = lds[(rv * 4 + 2) * P + c];
        o.w = lds[(rv * 4 + 3) * P + c];
      } else {
        const uint16_t* h = reinterpret_cast<const uint16_t*>(lds);
        uint32_t e[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) e[j] = h[(rv * 8 + j) * (2 * P) + c];
        o.x = e[0] | (e[1] << 16);
        o.y = e[2] | (e[3] << 16);
        o.z = e[4] | (e[5] << 16);
        o.w = e[6] | (e[7] << 16);
      }
      __builtin_nontemporal_store(
          o, reinterpret_cast<tr_u32x4*>(dst + ((c0 + c) * dst_stride + r0) * ES + rv * 16));
    }
  } else {
    // edge tiles and unaligned arrays: one element at a time, still through LDS so both sides stay coalesced
    for (int i = tid; i < TILE * TILE; i += 256) {
      const int row = i / TILE, col = i % TILE;
      if (r0 + row < rows && c0 + col < cols) {
        const char* p = src + ((r0 + row) * src_stride + c0 + col) * ES;
        if constexpr (ES == 4) {
          lds[row * P + col] = *reinterpret_cast<const uint32_t*>(p);
        } else {
          reinterpret_cast<uint16_t*>(lds)[row * (2 * P) + col] = *reinterpret_cast<const uint16_t*>(p);
        }
      }
    }
    __syncthreads();
    for (int i = tid; i < TILE * TILE; i += 256) {
      const int col = i / TILE, row = i % TILE;
      if (r0 + row < rows && c0 + col < cols) {
        char* p = dst + ((c0 + col) * dst_stride + r0 + row) * ES;
        if constexpr (ES == 4) {
          *reinterpret_cast<uint32_t*>(p) = lds[row * P + col];
        } else {
          *reinterpret_cast<uint16_t*>(p) = reinterpret_cast<const uint16_t*>(lds)[row * (2 * P) + col];
        }
      }
    }
  }
}

}  // namespace vrl
