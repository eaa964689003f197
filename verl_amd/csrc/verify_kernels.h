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

// ---- the same rule with 16-byte accesses ---------------------------------------------------------------------------
// A lane owns groups of 4 consecutive tokens that are aligned in the GLOBAL token index (so every full group is one
// 128-bit load per fp32 array, one 32-bit load of the mask, one 32-bit store of accept, whatever the sequence's first
// row is); the groups at a sequence's two ends that it shares with its neighbours are handled element by element.
// kVecGroups groups per lane are requested before any is used: a sequence of up to WAVES * 64 * 16 tokens (16384 for
// the 16-wavefront workgroup) costs one memory round trip, and its validity bits then stay in registers, so the count
// of valid tokens before the cut and the truncated mask need no second look at the mask. Longer sequences take more
// trips and finish with the element-wise loops of verify_sequence. Results are the same integers either way.
typedef float vf32x4 __attribute__((ext_vector_type(4)));
typedef long long vi64x2 __attribute__((ext_vector_type(2)));

constexpr int kVecGroups = 4;

// bits k < 4 with lo <= base + k < hi
__device__ __forceinline__ unsigned nibble_in_range(int64_t base, int64_t lo, int64_t hi) {
  unsigned n = 0;
#pragma unroll
  for (int k = 0; k < 4; ++k) n |= ((base + k >= lo) && (base + k < hi)) ? (1u << k) : 0u;
  return n;
}

// bits k < 4 whose in-sequence position pos0 + k lies before the cut
__device__ __forceinline__ unsigned nibble_before(int64_t pos0, int cut) {
  const int64_t room = static_cast<int64_t>(cut) - pos0;
  return room >= 4 ? 0xFu : (room <= 0 ? 0u : ((1u << static_cast<int>(room)) - 1u));
}

// 4 flag bits -> 4 bytes of 0 / 1
__device__ __forceinline__ uint32_t nibble_to_bytes(unsigned n) {
  return (n & 1u) | ((n & 2u) << 7) | ((n & 4u) << 14) | ((n & 8u) << 21);
}

__device__ __forceinline__ int wave_sum_int(int v) {
#pragma unroll
  for (int sh = 1; sh < 64; sh <<= 1) v += __shfl_xor(v, sh);
  return v;
}

// Needs 16-byte aligned logp_new / logp_old / log_u / draft_ids / out_ids and 4-byte aligned mask / accept / out_mask
// (the host checks and takes verify_sequence otherwise).
template <int WAVES>
__device__ __forceinline__ void verify_sequence_vec(const VerifyArgs& v, int64_t b) {
  constexpr int NTHR = WAVES * 64;
  constexpr int kG = kVecGroups;
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const SeqSpan sp = seq_span(v.cu_seqlens, b, v.T, v.n_tokens, v.err_flag);
  const int64_t s = sp.start, e = sp.start + sp.len;
  const int64_t q0 = s >> 2;                                          // first group of 4 (global index / 4)
  const int64_t n_groups = sp.len > 0 ? ((e + 3) >> 2) - q0 : 0;
  const bool one_trip = n_groups <= static_cast<int64_t>(NTHR) * kG;  // uniform over the workgroup

  int first = kNoReject;  // wave-uniform, as in verify_sequence
  int last_valid = 0;     // wave-uniform
  int near = 0;           // per lane
  unsigned valn[kG];      // validity bits of this lane's groups in the last trip
#pragma unroll
  for (int j = 0; j < kG; ++j) valn[j] = 0;

  for (int64_t qb = 0; qb < n_groups; qb += static_cast<int64_t>(NTHR) * kG) {
    vf32x4 ln[kG], lo[kG], lu[kG];
    uint32_t mk[kG];    // 4 mask bytes
    unsigned inb[kG];   // which of the group's 4 tokens belong to this sequence
#pragma unroll
    for (int j = 0; j < kG; ++j) {
      const int64_t qi = qb + static_cast<int64_t>(j) * NTHR + tid;
      const int64_t g0 = (q0 + qi) << 2;
      inb[j] = qi < n_groups ? nibble_in_range(g0, s, e) : 0u;
      ln[j] = lo[j] = lu[j] = vf32x4{0.f, 0.f, 0.f, 0.f};
      mk[j] = 0;
      if (inb[j] == 0xFu) {
        ln[j] = *reinterpret_cast<const vf32x4*>(v.logp_new + g0);
        lo[j] = *reinterpret_cast<const vf32x4*>(v.logp_old + g0);
        lu[j] = *reinterpret_cast<const vf32x4*>(v.log_u + g0);
        mk[j] = (v.mask != nullptr) ? *reinterpret_cast<const uint32_t*>(v.mask + g0) : 0x01010101u;
      } else if (inb[j] != 0u) {
#pragma unroll
        for (int k = 0; k < 4; ++k) {
          if ((inb[j] >> k) & 1u) {
            ln[j][k] = v.logp_new[g0 + k];
            lo[j][k] = v.logp_old[g0 + k];
            lu[j][k] = v.log_u[g0 + k];
            const uint32_t m = (v.mask != nullptr) ? static_cast<uint32_t>(v.mask[g0 + k]) : 1u;
            mk[j] |= m << (8 * k);
          }
        }
      }
    }
#pragma unroll
    for (int j = 0; j < kG; ++j) {
      const int64_t cbase = qb + static_cast<int64_t>(j) * NTHR;
      if (cbase >= n_groups) break;  // uniform over the workgroup
      unsigned rejn = 0, vn = 0, nearn = 0, accn = 0;
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        const float d = ln[j][k] - lo[j][k];
        const float tau = lu[j][k] + v.thresh_offset;
        const bool valid = (((inb[j] >> k) & 1u) != 0u) && (((mk[j] >> (8 * k)) & 0xffu) != 0u);
        const bool ok = d >= tau;
        const bool close = valid && (__builtin_fabsf(d - tau) < v.near_eps);
        rejn |= (valid && !ok) ? (1u << k) : 0u;
        vn |= valid ? (1u << k) : 0u;
        nearn |= close ? (1u << k) : 0u;
        accn |= (valid && ok) ? (1u << k) : 0u;
      }
      valn[j] = vn;
      const int64_t g0 = (q0 + cbase + tid) << 2;
      if (inb[j] == 0xFu) {
        *reinterpret_cast<uint32_t*>(v.accept + g0) = nibble_to_bytes(accn);
      } else if (inb[j] != 0u) {
#pragma unroll
        for (int k = 0; k < 4; ++k)
          if ((inb[j] >> k) & 1u) v.accept[g0 + k] = static_cast<uint8_t>((accn >> k) & 1u);
      }
      near += __builtin_popcount(nearn);
      const unsigned long long rb = __ballot(rejn != 0u);
      const unsigned long long vb = __ballot(vn != 0u);
      // in-sequence position of element 0 of lane 0's group (down to -3 for the group a sequence shares with the one before)
      const int64_t pw = ((q0 + cbase + static_cast<int64_t>(wave) * 64) << 2) - s;
      if (rb != 0ull && first == kNoReject) {
        const int fl = __builtin_ctzll(rb);
        const unsigned n = static_cast<unsigned>(__builtin_amdgcn_readlane(static_cast<int>(rejn), fl));
        first = static_cast<int>(pw + 4 * fl + __builtin_ctz(n));
      }
      if (vb != 0ull) {
        const int ll = 63 - __builtin_clzll(vb);
        const unsigned n = static_cast<unsigned>(__builtin_amdgcn_readlane(static_cast<int>(vn), ll));
        last_valid = static_cast<int>(pw + 4 * ll + (32 - __builtin_clz(n)));
      }
    }
  }
  near = wave_sum_int(near);

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
    if (one_trip) {
#pragma unroll
      for (int j = 0; j < kG; ++j) {
        const int64_t pos0 = ((q0 + static_cast<int64_t>(j) * NTHR + tid) << 2) - s;
        cnt += __builtin_popcount(valn[j] & nibble_before(pos0, f));
      }
      cnt = wave_sum_int(cnt);
    } else {
      for (int64_t base = 0; base < f; base += NTHR) {
        const int64_t i = base + tid;
        const bool m = (i < f) && (v.mask[sp.start + i] != 0);
        cnt += __builtin_popcountll(__ballot(m));
      }
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
  if (v.out_ids == nullptr) return;   // behind the last barrier
  if (!one_trip) {
    truncate_span<WAVES>(sp, f, v.draft_ids, v.mask, v.pad_id, v.out_ids, v.out_mask);
    return;
  }
#pragma unroll
  for (int j = 0; j < kG; ++j) {
    const int64_t qi = static_cast<int64_t>(j) * NTHR + tid;
    if (qi >= n_groups) continue;
    const int64_t g0 = (q0 + qi) << 2;
    const unsigned in = nibble_in_range(g0, s, e);
    const unsigned keep = in & nibble_before(g0 - s, f);
    if (in == 0xFu) {
      vi64x2 a = {v.pad_id, v.pad_id}, c = {v.pad_id, v.pad_id};
      if (keep == 0xFu) {
        a = *reinterpret_cast<const vi64x2*>(v.draft_ids + g0);
        c = *reinterpret_cast<const vi64x2*>(v.draft_ids + g0 + 2);
      } else if (keep != 0u) {   // the group that holds the cut: keep is 1, 3 or 7
        a[0] = v.draft_ids[g0];
        if (keep & 2u) a[1] = v.draft_ids[g0 + 1];
        if (keep & 4u) c[0] = v.draft_ids[g0 + 2];
      }
      *reinterpret_cast<vi64x2*>(v.out_ids + g0) = a;
      *reinterpret_cast<vi64x2*>(v.out_ids + g0 + 2) = c;
      *reinterpret_cast<uint32_t*>(v.out_mask + g0) = nibble_to_bytes(valn[j] & keep);
    } else {
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        if ((in >> k) & 1u) {
          const bool kp = ((keep >> k) & 1u) != 0u;
          v.out_ids[g0 + k] = kp ? v.draft_ids[g0 + k] : v.pad_id;
          v.out_mask[g0 + k] = static_cast<uint8_t>((valn[j] & keep) >> k & 1u);
        }
      }
    }
  }
}

template <int WAVES>
__global__ __launch_bounds__(WAVES * 64) void spec_verify_vec_kernel(const VerifyArgs v) {
  verify_sequence_vec<WAVES>(v, blockIdx.x);
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
