// Packed per-token values -> padded (B, T_out) response block, shifted left by
// one token: the model output at position p scores token p+1, so the response
// tokens of a sequence that ends at row `end` with `r` response tokens are
// scored by rows [end - r - 1, end - 1).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace vrl {

// Offsets read from device memory are held to the size of `values` before anything is indexed with them: a span must
// lie in [0, n_tokens], be non-decreasing, start at 0 for the first sequence and end at n_tokens for the last
// (workgroup b of a grid of B). A sequence whose span fails contributes nothing and sets VRL_FLAG_SEQ_RANGE (4).
__device__ __forceinline__ bool span_in_range(int64_t begin, int64_t end, int64_t b, int64_t n_tokens) {
  return (begin >= 0) && (end <= n_tokens) && (end >= begin) && (b != 0 || begin == 0) &&
         (b + 1 != static_cast<int64_t>(gridDim.x) || end == n_tokens);
}

// grid.x = B, block = 256. Sequence b owns packed rows [cu[b], cu[b+1]).
__global__ __launch_bounds__(256) void response_slice_kernel(
    const float* __restrict__ values, const int64_t* __restrict__ cu_seqlens,
    const int64_t* __restrict__ response_lens, int64_t n_tokens, int64_t T_out, float* __restrict__ out,
    int32_t* err_flag) {
  const int64_t b = blockIdx.x;
  const int64_t begin = cu_seqlens[b];
  const int64_t end = cu_seqlens[b + 1];
  const int64_t r = response_lens[b];
  const int64_t first = end - r - 1;
  // offsets must partition [0, n_tokens], as the reference asserts (sequence_offsets[-1] == values.shape[0])
  const bool span_ok = span_in_range(begin, end, b, n_tokens);
  if (!span_ok && threadIdx.x == 0) atomicOr(err_flag, 4);
  // the reference asserts prompt_len > 0 (first >= begin) and pads up to T_out (r <= T_out)
  const bool ok = span_ok && (r >= 0) && (r <= T_out) && (first >= begin);
  if (span_ok && !ok && threadIdx.x == 0) atomicOr(err_flag, 2);
  float* dst = out + b * T_out;
  for (int64_t j = threadIdx.x; j < T_out; j += 256) dst[j] = (ok && j < r) ? values[first + j] : 0.f;
}

// Packed in, packed out: the response positions of sequence b, shifted like above, go to
// out[out_offsets[b] .. out_offsets[b] + r). grid.x = B, block = 256.
__global__ __launch_bounds__(256) void response_pack_kernel(
    const float* __restrict__ values, const int64_t* __restrict__ cu_seqlens,
    const int64_t* __restrict__ response_lens, const int64_t* __restrict__ out_offsets, int64_t n_tokens,
    int64_t out_total, float* __restrict__ out, int32_t* err_flag) {
  const int64_t b = blockIdx.x;
  const int64_t begin = cu_seqlens[b];
  const int64_t end = cu_seqlens[b + 1];
  const int64_t r = response_lens[b];
  const int64_t first = end - r - 1;
  const int64_t o = out_offsets[b];
  // the output window must be the caller's prefix sum of the response lengths and lie inside the output
  const bool span_ok = span_in_range(begin, end, b, n_tokens);
  const bool ok = span_ok && (r >= 0) && (first >= begin) && (o >= 0) && (o <= out_total - r) &&
                  (out_offsets[b + 1] - o == r);
  if (!ok) {
    if (threadIdx.x == 0) atomicOr(err_flag, span_ok ? 2 : 4);
    return;  // no barrier follows
  }
  for (int64_t j = threadIdx.x; j < r; j += 256) out[o + j] = values[first + j];
}

}  // namespace vrl
