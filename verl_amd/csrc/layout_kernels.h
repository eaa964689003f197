// Packed per-token values -> padded (B, T_out, ...) response block, shifted left by
// one token: the model output at position p scores token p+1, so the response
// tokens of a sequence that ends at row `end` with `r` response tokens are
// scored by rows [end - r - 1, end - 1).
//
// A token's value is a row of `row_bytes` bytes (one element of any size, or the product of trailing dimensions times
// the element size: top-k log-probs, hidden vectors), copied bit for bit; the padding is zero bytes. The kernels move
// units of U bytes, U the largest of 16, 8, 4, 2, 1 that divides row_bytes and the alignment of both arrays.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace vrl {

template <int U>
struct CopyUnit;
template <>
struct CopyUnit<1> {
  typedef uint8_t type;
};
template <>
struct CopyUnit<2> {
  typedef uint16_t type;
};
template <>
struct CopyUnit<4> {
  typedef uint32_t type;
};
template <>
struct CopyUnit<8> {
  typedef uint2 type;
};
template <>
struct CopyUnit<16> {
  typedef uint4 type;
};

constexpr int kSliceThreads = 256;
constexpr int kSliceUnitsPerThread = 8;
constexpr int64_t kSliceChunk = static_cast<int64_t>(kSliceThreads) * kSliceUnitsPerThread;   // units per workgroup

// Offsets read from device memory are held to the size of `values` before anything is indexed with them: a span must
// lie in [0, n_tokens], be non-decreasing, start at 0 for the first sequence and end at n_tokens for the last
// (workgroup column b of a grid of B). A sequence whose span fails contributes nothing and sets VRL_FLAG_SEQ_RANGE (4).
__device__ __forceinline__ bool span_in_range(int64_t begin, int64_t end, int64_t b, int64_t n_tokens) {
  return (begin >= 0) && (end <= n_tokens) && (end >= begin) && (b != 0 || begin == 0) &&
         (b + 1 != static_cast<int64_t>(gridDim.x) || end == n_tokens);
}

// grid = (B, chunks of kSliceChunk units of a sequence's T_out * row_units output units), block = 256.
// Sequence b owns packed rows [cu[b], cu[b+1]).
template <int U>
__global__ __launch_bounds__(kSliceThreads) void response_slice_kernel(
    const char* __restrict__ values, int64_t row_units, const int64_t* __restrict__ cu_seqlens,
    const int64_t* __restrict__ response_lens, int64_t n_tokens, int64_t T_out, char* __restrict__ out,
    int32_t* err_flag) {
  typedef typename CopyUnit<U>::type unit_t;
  const int64_t b = blockIdx.x;
  const int64_t begin = cu_seqlens[b];
  const int64_t end = cu_seqlens[b + 1];
  const int64_t r = response_lens[b];
  const int64_t first = end - r - 1;
  // offsets must partition [0, n_tokens], as the reference asserts (sequence_offsets[-1] == values.shape[0])
  const bool span_ok = span_in_range(begin, end, b, n_tokens);
  const bool reporter = threadIdx.x == 0 && blockIdx.y == 0;
  if (!span_ok && reporter) atomicOr(err_flag, 4);
  // the reference asserts prompt_len > 0 (first >= begin) and pads up to T_out (r <= T_out)
  const bool ok = span_ok && (r >= 0) && (r <= T_out) && (first >= begin);
  if (span_ok && !ok && reporter) atomicOr(err_flag, 2);
  const int64_t total = T_out * row_units;
  const int64_t copy = ok ? r * row_units : 0;
  const unit_t* src = reinterpret_cast<const unit_t*>(values) + (ok ? first * row_units : 0);
  unit_t* dst = reinterpret_cast<unit_t*>(out) + b * total;
  const int64_t u0 = static_cast<int64_t>(blockIdx.y) * kSliceChunk;
  const unit_t zero = {};
#pragma unroll
  for (int k = 0; k < kSliceUnitsPerThread; ++k) {
    const int64_t u = u0 + static_cast<int64_t>(k) * kSliceThreads + threadIdx.x;
    if (u < total) dst[u] = (u < copy) ? src[u] : zero;
  }
}

// Packed in, packed out: the response positions of sequence b, shifted like above, go to
// rows [out_offsets[b], out_offsets[b] + r) of out. grid = (B, chunks of max_rows * row_units units), block = 256.
template <int U>
__global__ __launch_bounds__(kSliceThreads) void response_pack_kernel(
    const char* __restrict__ values, int64_t row_units, const int64_t* __restrict__ cu_seqlens,
    const int64_t* __restrict__ response_lens, const int64_t* __restrict__ out_offsets, int64_t n_tokens,
    int64_t out_total, char* __restrict__ out, int32_t* err_flag) {
  typedef typename CopyUnit<U>::type unit_t;
  const int64_t b = blockIdx.x;
  const int64_t begin = cu_seqlens[b];
  const int64_t end = cu_seqlens[b + 1];
  const int64_t r = response_lens[b];
  const int64_t first = end - r - 1;
  const int64_t o = out_offsets[b];
  // the output window must be the caller's prefix sum of the response lengths and lie inside the output
  const bool span_ok = span_in_range(begin, end, b, n_tokens);
  const bool ok = span_ok && (r >= 0) && (first >= begin) && (o >= 0) && (o <= out_total - r) &&
                  (out_offsets[b + 1] - o == r) &&
                  (b + 1 != static_cast<int64_t>(gridDim.x) || out_offsets[b + 1] == out_total);
  if (!ok) {
    if (threadIdx.x == 0 && blockIdx.y == 0) atomicOr(err_flag, span_ok ? 2 : 4);
    return;  // no barrier follows
  }
  const int64_t copy = r * row_units;
  const unit_t* src = reinterpret_cast<const unit_t*>(values) + first * row_units;
  unit_t* dst = reinterpret_cast<unit_t*>(out) + o * row_units;
  // the grid's second dimension is sized for the longest window the output could hold; this sequence's ends at `copy`
  for (int64_t u0 = static_cast<int64_t>(blockIdx.y) * kSliceChunk; u0 < copy;
       u0 += static_cast<int64_t>(gridDim.y) * kSliceChunk) {
#pragma unroll
    for (int k = 0; k < kSliceUnitsPerThread; ++k) {
      const int64_t u = u0 + static_cast<int64_t>(k) * kSliceThreads + threadIdx.x;
      if (u < copy) dst[u] = src[u];
    }
  }
}

// One value per sequence -> one value per token of the packed batch: out[t] = values[b] for the sequence b that holds
// token t (cu_seqlens[b] <= t < cu_seqlens[b+1]). One thread per token finds its sequence by bisection over the
// offsets (every index stays in [0, B], whatever they hold) and writes exactly one element; a token that no sequence
// holds gets 0 and sets VRL_FLAG_SEQ_RANGE (4), and so do offsets that do not start at 0, end at n_tokens or decrease
// (threads 0 .. B check one entry each). grid = ceil(max(n_tokens, B + 1) / 256), block = 256, B >= 1.
__global__ __launch_bounds__(kSliceThreads) void expand_per_sequence_kernel(
    const float* __restrict__ values, const int64_t* __restrict__ cu_seqlens, int64_t B, int64_t n_tokens,
    float* __restrict__ out, int32_t* err_flag) {
  const int64_t t = static_cast<int64_t>(blockIdx.x) * kSliceThreads + threadIdx.x;
  bool bad = false;
  if (t <= B) {
    const int64_t c = cu_seqlens[t];
    bad = (t == 0 && c != 0) || (t == B && c != n_tokens) || (t < B && cu_seqlens[t + 1] < c);
  }
  if (t < n_tokens) {
    int64_t lo = 0, hi = B;   // the largest b < B with cu_seqlens[b] <= t lies in [lo, hi)
    while (hi - lo > 1) {
      const int64_t mid = (lo + hi) >> 1;
      if (cu_seqlens[mid] <= t) lo = mid; else hi = mid;
    }
    const bool held = cu_seqlens[lo] <= t && t < cu_seqlens[lo + 1];
    out[t] = held ? values[lo] : 0.f;
    bad = bad || !held;
  }
  if (bad) atomicOr(err_flag, 4);
}

}  // namespace vrl
