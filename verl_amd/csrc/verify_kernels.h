// SPEC-RL draft verification: one workgroup per sequence.
//
// Per token: d = logp_new - logp_old, tau = log_u + thresh_offset, both single
// fp32 operations (no multiply, so nothing can be contracted), accept iff the
// token is valid and d >= tau. Each wavefront turns its 64 predicates into a
// ballot; the first set bit of the first non-empty "rejected" ballot is that
// wavefront's earliest rejection, and the minimum over wavefronts (through
// LDS) is the sequence's. Counts come from popcounts of ballots, so every
// per-sequence result is produced without atomics and is deterministic.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace vrl {

constexpr int kNoReject = 0x7fffffff;

struct SeqSpan {
  int64_t start;
  int64_t len;
};

constexpr int kFlagSeqRange = 4;  // VRL_FLAG_SEQ_RANGE

// Rows [start, start + len) of sequence b (workgroup b of a grid of B). Packed offsets come from device memory the
// host cannot see, so they are held to the arrays' size here: a span is cut to [0, n_tokens] (an inverted one to
// nothing), and offsets that are not a partition of [0, n_tokens] (first != 0, last != n_tokens, decreasing, out of
// range) set VRL_FLAG_SEQ_RANGE. Nothing outside the per-token arrays is ever touched.
__device__ __forceinline__ SeqSpan seq_span(const int64_t* cu_seqlens, int64_t b, int64_t T, int64_t n_tokens,
                                            int32_t* err_flag) {
  SeqSpan s;
  if (cu_seqlens != nullptr) {
    int64_t lo = cu_seqlens[b];
    int64_t hi = cu_seqlens[b + 1];
    const bool bad = (lo < 0) || (hi > n_tokens) || (hi < lo) || (b == 0 && lo != 0) ||
                     (b + 1 == static_cast<int64_t>(gridDim.x) && hi != n_tokens);
    if (bad && threadIdx.x == 0 && err_flag != nullptr) atomicOr(err_flag, kFlagSeqRange);
    lo = lo < 0 ? 0 : (lo > n_tokens ? n_tokens : lo);
    hi = hi < lo ? lo : (hi > n_tokens ? n_tokens : hi);
    s.start = lo;
    s.len = hi - lo;
  } else {
    s.start = b * T;
    s.len = T;
  }
  return s;
}

template <int WAVES>
__device__ __forceinline__ void truncate_span(const SeqSpan sp, int first, const int64_t* draft_ids,
                                              const uint8_t* mask, int64_t pad_id, int64_t* out_ids,
                                              uint8_t* out_mask) {
  constexpr int NTHR = WAVES * 64;
  // Positions at or after the cut need no load at all.
#pragma unroll 4
  for (int64_t i = threadIdx.x; i < sp.len; i += NTHR) {
    const bool keep = i < first;
    const int64_t g = sp.start + i;
    int64_t id = pad_id;
    uint8_t mv = 0;
    if (keep) {
      id = draft_ids[g];
      mv = (mask != nullptr) ? static_cast<uint8_t>(mask[g] != 0) : static_cast<uint8_t>(1);
    }
    out_ids[g] = id;
    out_mask[g] = mv;
  }
}

struct VerifyArgs {
  const float* logp_new;
  const float* logp_old;
  const float* log_u;
  const uint8_t* mask;
  const int64_t* cu_seqlens;
  int64_t B;
  int64_t T;
  int64_t n_tokens;   // length of every per-token array
  int32_t* err_flag;  // VRL_FLAG_SEQ_RANGE lands here (packed layout)
  float thresh_offset;
  float near_eps;
  uint8_t* accept;
  int32_t* first_reject;
  int32_t* prefix_len;
  int32_t* near_count;
  const int64_t* draft_ids;
  int64_t pad_id;
  int64_t* out_ids;
  uint8_t* out_mask;
};

// The whole workgroup (WAVES*64 threads, all of them) verifies sequence b.
template <int WAVES>
__device__ __forceinline__ void verify_sequence(const VerifyArgs& v, int64_t b) {
  constexpr int NTHR = WAVES * 64;
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const SeqSpan sp = seq_span(v.cu_seqlens, b, v.T, v.n_tokens, v.err_flag);

  // wave-uniform running results
  int first = kNoReject;  // earliest rejected position seen by this wavefront
  int last_valid = 0;     // one past the last valid position seen by this wavefront
  int near = 0;

  // kChunks chunks of NTHR tokens per trip, all loads of a trip issued before any is used, so a long
  // sequence costs len / (kChunks * NTHR) memory round trips instead of len / NTHR.
  constexpr int kChunks = 4;
  for (int64_t base = 0; base < sp.len; base += static_cast<int64_t>(NTHR) * kChunks) {
    float ln[kChunks], lo[kChunks], lu[kChunks];
    uint8_t mk[kChunks];
    bool in[kChunks];
#pragma unroll
    for (int j = 0; j < kChunks; ++j) {
      const int64_t i = base + static_cast<int64_t>(j) * NTHR + tid;
      in[j] = i < sp.len;
      ln[j] = lo[j] = lu[j] = 0.f;
      mk[j] = 0;
      if (in[j]) {
        const int64_t g = sp.start + i;
        ln[j] = v.logp_new[g];
        lo[j] = v.logp_old[g];
        lu[j] = v.log_u[g];
        mk[j] = (v.mask != nullptr) ? v.mask[g] : static_cast<uint8_t>(1);
      }
    }
#pragma unroll
    for (int j = 0; j < kChunks; ++j) {
      const int64_t cbase = base + static_cast<int64_t>(j) * NTHR;
      if (cbase >= sp.len) break;  // uniform over the workgroup
      const float d = ln[j] - lo[j];
      const float tau = lu[j] + v.thresh_offset;
      const bool valid = in[j] && (mk[j] != 0);
      const bool ok = d >= tau;
      const bool close = valid && (__builtin_fabsf(d - tau) < v.near_eps);
      if (in[j]) v.accept[sp.start + cbase + tid] = static_cast<uint8_t>(valid && ok);
      const unsigned long long rej = __ballot(valid && !ok);
      const unsigned long long val = __ballot(valid);
      const unsigned long long nr = __ballot(close);
      const int wbase = static_cast<int>(cbase) + wave * 64;
      if (rej != 0ull && first == kNoReject) first = wbase + __builtin_ctzll(rej);
      if (val != 0ull) last_valid = wbase + 64 - __builtin_clzll(val);
      near += __builtin_popcountll(nr);
    }
  }

  __shared__ int sm_first[WAVES];
  __shared__ int sm_last[WAVES];
  __shared__ int sm_near[WAVES];
  __shared__ int sm_cnt[WAVES];
  if (lane == 0) {
    sm_first[wave] = first;
    sm_last[wave] = last_valid;
    sm_near[wave] = near;
  }
  __syncthreads();
  int f = kNoReject, lv = 0, nc = 0;
#pragma unroll
  for (int w = 0; w < WAVES; ++w) {
    f = min(f, sm_first[w]);
    lv = max(lv, sm_last[w]);
    nc += sm_near[w];
  }
  if (f == kNoReject) f = lv;

  // valid tokens strictly before the first rejection
  int cnt = 0;
  if (v.mask != nullptr) {
    for (int64_t base = 0; base < f; base += NTHR) {
      const int64_t i = base + tid;
      const bool m = (i < f) && (v.mask[sp.start + i] != 0);
      cnt += __builtin_popcountll(__ballot(m));
    }
  }
  if (lane == 0) sm_cnt[wave] = cnt;
  __syncthreads();
  if (tid == 0) {
    int total = f;
    if (v.mask != nullptr) {
      total = 0;
#pragma unroll
      for (int w = 0; w < WAVES; ++w) total += sm_cnt[w];
    }
    v.first_reject[b] = f;
    v.prefix_len[b] = total;
    v.near_count[b] = nc;
  }
  if (v.out_ids != nullptr) truncate_span<WAVES>(sp, f, v.draft_ids, v.mask, v.pad_id, v.out_ids, v.out_mask);
}

// grid.x = B, block = WAVES*64. No thread leaves before the last barrier.
template <int WAVES>
__global__ __launch_bounds__(WAVES * 64) void spec_verify_kernel(const VerifyArgs v) {
  verify_sequence<WAVES>(v, blockIdx.x);
}

template <int WAVES>
__global__ __launch_bounds__(WAVES * 64) void truncate_draft_kernel(
    const int64_t* __restrict__ draft_ids, const uint8_t* __restrict__ mask,
    const int64_t* __restrict__ cu_seqlens, int64_t T, int64_t n_tokens, const int32_t* __restrict__ first_reject,
    int64_t pad_id, int64_t* __restrict__ out_ids, uint8_t* __restrict__ out_mask, int32_t* err_flag) {
  const int64_t b = blockIdx.x;
  const SeqSpan sp = seq_span(cu_seqlens, b, T, n_tokens, err_flag);
  truncate_span<WAVES>(sp, first_reject[b], draft_ids, mask, pad_id, out_ids, out_mask);
}

}  // namespace vrl
