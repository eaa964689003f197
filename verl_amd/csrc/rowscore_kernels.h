// Fused vocab-row kernel for gfx950: one pass over a row of logits yields the
// label log-probability and the Shannon entropy of softmax(row / T).
//
// Arithmetic. Everything is kept in the log2 domain so the inner loop is
//   d = fma(x, c, -m);  e = v_exp_f32(d);  s += e;  t = fma(e, d, t)
// with c = log2(e) / T and m a running shift (the largest x*c this thread has
// seen, refreshed once per register batch). A partial result is the triple
// (m, s, t) with  s = sum 2^(y - m),  t = sum 2^(y - m) * (y - m),  y = x*c.
// Two partials are merged by bringing both to the larger shift M:
//   alpha = 2^(m - M);  s' = alpha*s;  t' = alpha*(t + (m - M)*s).
// At the end  logsumexp = ln2*(M + log2 S),  logprob = ln2*((y_label - M) - log2 S),
// entropy = ln2*(log2 S - T/S)  (the shift cancels, nothing large is subtracted).
// The optional sum of squared probabilities carries q = sum 2^(2(y-m)), merged with
// alpha^2, and ends as Q/S^2.
//
// Mapping. One workgroup of WAVES wavefronts owns one row (or, when there are
// too few rows to fill the chip, one slice of a row; a second small kernel then
// merges the slices). A register batch is
// U 128-bit loads per lane; wave w of the group reads the w-th contiguous
// U KiB slice of each WAVES*U KiB block of the row, so every load instruction
// is one fully coalesced 1 KiB request and a lane's U loads differ only in the
// instruction's immediate offset. Lanes reduce over the 64-lane wavefront with
// DPP row operations + readlane, wavefronts through LDS.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace vrl {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

constexpr float kLog2e = 1.44269504088896340736f;
constexpr double kLn2d = 0.693147180559945309417232;
constexpr float kMinTemperature = 1e-8f;  // verl/workers/engine/fsdp/transformer_impl.py:1357 clamp(min=1e-8)

__device__ __forceinline__ float neg_inf() { return -__builtin_huge_valf(); }
__device__ __forceinline__ float pos_inf() { return __builtin_huge_valf(); }
__device__ __forceinline__ float quiet_nan() { return __builtin_nanf(""); }
__device__ __forceinline__ float hw_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

struct Part {
  float m;  // shift, log2 domain; -inf while nothing finite has been seen
  float s;  // sum 2^(y-m)
  float t;  // sum 2^(y-m)*(y-m)
  float q;  // sum 2^(2(y-m)), only maintained when the sum of squared probabilities is asked for
};

// Bring p to the shift M >= p.m. A partial that has seen nothing finite
// (m == -inf, s == 0) stays zero instead of producing 0*inf.
__device__ __forceinline__ void rescale(Part& p, float M) {
  const bool dead = (p.m == neg_inf());
  const float dm = dead ? 0.f : p.m - M;
  const float alpha = dead ? 0.f : hw_exp2(dm);
  p.t = alpha * (p.t + dm * p.s);
  p.s = alpha * p.s;
  p.q = (alpha * alpha) * p.q;
  p.m = M;
}

// ---- element types -------------------------------------------------------
template <int DT>
struct Elem;

template <>
struct Elem<0> {  // VRL_F32
  static constexpr int kBytes = 4;
  static constexpr int kPerVec = 4;
  __device__ static __forceinline__ void unpack(const u32x4& v, float* x) {
    x[0] = __uint_as_float(v.x);
    x[1] = __uint_as_float(v.y);
    x[2] = __uint_as_float(v.z);
    x[3] = __uint_as_float(v.w);
  }
  __device__ static __forceinline__ float load1(const char* rowp, int64_t idx) {
    return reinterpret_cast<const float*>(rowp)[idx];
  }
};

template <>
struct Elem<1> {  // VRL_BF16: the upper half of an fp32
  static constexpr int kBytes = 2;
  static constexpr int kPerVec = 8;
  __device__ static __forceinline__ void unpack(const u32x4& v, float* x) {
    x[0] = __uint_as_float(v.x << 16);
    x[1] = __uint_as_float(v.x & 0xffff0000u);
    x[2] = __uint_as_float(v.y << 16);
    x[3] = __uint_as_float(v.y & 0xffff0000u);
    x[4] = __uint_as_float(v.z << 16);
    x[5] = __uint_as_float(v.z & 0xffff0000u);
    x[6] = __uint_as_float(v.w << 16);
    x[7] = __uint_as_float(v.w & 0xffff0000u);
  }
  __device__ static __forceinline__ float load1(const char* rowp, int64_t idx) {
    return __uint_as_float(static_cast<uint32_t>(reinterpret_cast<const uint16_t*>(rowp)[idx]) << 16);
  }
};

template <>
struct Elem<2> {  // VRL_F16: IEEE half
  typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
  typedef float f32x2v __attribute__((ext_vector_type(2)));
  static constexpr int kBytes = 2;
  static constexpr int kPerVec = 8;
  __device__ static __forceinline__ void unpack2(uint32_t w, float* x) {
    const f32x2v f = __builtin_convertvector(__builtin_bit_cast(f16x2, w), f32x2v);
    x[0] = f.x;
    x[1] = f.y;
  }
  __device__ static __forceinline__ void unpack(const u32x4& v, float* x) {
    unpack2(v.x, x);
    unpack2(v.y, x + 2);
    unpack2(v.z, x + 4);
    unpack2(v.w, x + 6);
  }
  __device__ static __forceinline__ float load1(const char* rowp, int64_t idx) {
    return static_cast<float>(reinterpret_cast<const _Float16*>(rowp)[idx]);
  }
};

// ---- temperature ---------------------------------------------------------
// EXACT = false: y = x * c with c = log2e / T folded into one constant.
// EXACT = true : q = RN(x / T) first (what `logits / temperature` gives per
//                element in fp32), then y = q * log2e. The quotient uses the
//                reciprocal + one fma correction, which is the correctly
//                rounded quotient whenever r is the correctly rounded 1/T.
template <bool EXACT>
struct Scale {
  float c;   // multiplier applied by the fma in the inner loop
  float T;   // clamped temperature
  float r;   // RN(1/T)
  __device__ __forceinline__ float pre(float x) const {
    if constexpr (EXACT) {
      const float q0 = x * r;
      const float rem = __builtin_fmaf(-q0, T, x);
      const float q = __builtin_fmaf(rem, r, q0);
      // inf / T must stay inf (rem is NaN there), and so must NaN stay NaN
      return (__builtin_fabsf(q0) == pos_inf()) ? q0 : q;
    } else {
      return x;
    }
  }
};

// ---- one register batch --------------------------------------------------
template <int N, bool EXACT, bool WANT_Q>
__device__ __forceinline__ void accumulate(Part& a, float* x, const Scale<EXACT>& sc) {
  if constexpr (EXACT) {
#pragma unroll
    for (int i = 0; i < N; ++i) x[i] = sc.pre(x[i]);
  }
  float bm = x[0];
#pragma unroll
  for (int i = 1; i < N; ++i) bm = __builtin_fmaxf(bm, x[i]);
  const float bm2 = bm * sc.c;
  if (bm2 > a.m) {  // strictly greater, so bm2 > -inf
    rescale(a, bm2);
  }
  // While only -inf has been seen the shift must stay finite: -inf - (-inf) is NaN.
  const float sub = (a.m == neg_inf()) ? 0.f : a.m;
  float ps = 0.f, pt = 0.f, pq = 0.f;
#pragma unroll
  for (int i = 0; i < N; ++i) {
    const float d = __builtin_fmaf(x[i], sc.c, -sub);
    const float e = hw_exp2(d);
    ps += e;
    pt = __builtin_fmaf(e, d, pt);
    if constexpr (WANT_Q) pq = __builtin_fmaf(e, e, pq);
  }
  a.s += ps;
  a.t += pt;
  if constexpr (WANT_Q) a.q += pq;
}

// ---- wavefront reductions (DPP within rows of 16 lanes, readlane across) ---
template <int CTRL>
__device__ __forceinline__ float dpp_mov(float v) {
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xF, 0xF, false));
}
__device__ __forceinline__ float lane_value(float v, int lane) {
  return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), lane));
}
__device__ __forceinline__ float wave_max(float v) {
  v = __builtin_fmaxf(v, dpp_mov<0xB1>(v));   // quad_perm [1,0,3,2]
  v = __builtin_fmaxf(v, dpp_mov<0x4E>(v));   // quad_perm [2,3,0,1]
  v = __builtin_fmaxf(v, dpp_mov<0x141>(v));  // row_half_mirror
  v = __builtin_fmaxf(v, dpp_mov<0x140>(v));  // row_mirror
  return __builtin_fmaxf(__builtin_fmaxf(lane_value(v, 0), lane_value(v, 16)),
                         __builtin_fmaxf(lane_value(v, 32), lane_value(v, 48)));
}
__device__ __forceinline__ float wave_sum(float v) {
  v += dpp_mov<0xB1>(v);
  v += dpp_mov<0x4E>(v);
  v += dpp_mov<0x141>(v);
  v += dpp_mov<0x140>(v);
  return (lane_value(v, 0) + lane_value(v, 16)) + (lane_value(v, 32) + lane_value(v, 48));
}

template <bool NT>
__device__ __forceinline__ u32x4 load_vec(const u32x4* p) {
  if constexpr (NT) {
    return __builtin_nontemporal_load(p);
  } else {
    return *p;
  }
}

// ---- a workgroup reduces elements [e_lo, e_hi) of one row -------------------
// Every thread of the workgroup must call this (it contains a barrier and DPP
// operations that need a full EXEC mask). The result is valid in thread 0.
template <int DT, int WAVES, int U, bool EXACT, bool NT, bool WANT_Q>
__device__ __forceinline__ Part block_reduce_range(const char* rowp, int64_t e_lo, int64_t e_hi,
                                                   const Scale<EXACT>& sc) {
  using E = Elem<DT>;
  constexpr int NTHR = WAVES * 64;
  constexpr int PV = E::kPerVec;
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;

  // Split the range into [head scalars][16-byte vectors][tail scalars].
  const int64_t count = e_hi - e_lo;
  const char* basep = rowp + e_lo * E::kBytes;
  const uintptr_t addr = reinterpret_cast<uintptr_t>(basep);
  int64_t head = static_cast<int64_t>(((16u - (addr & 15u)) & 15u) / E::kBytes);
  if (head > count) head = count;
  const int64_t nvec = (count - head) / PV;
  const int64_t tail0 = head + nvec * PV;
  const u32x4* vp = reinterpret_cast<const u32x4*>(basep + head * E::kBytes);

  Part a;
  a.m = neg_inf();
  a.s = 0.f;
  a.t = 0.f;
  a.q = 0.f;

  constexpr int64_t kBatchVecs = static_cast<int64_t>(NTHR) * U;
  const int64_t nfull = nvec / kBatchVecs;
  for (int64_t j = 0; j < nfull; ++j) {
    const u32x4* p = vp + (j * WAVES + wave) * (U * 64) + lane;
    u32x4 v[U];
#pragma unroll
    for (int u = 0; u < U; ++u) v[u] = load_vec<NT>(p + u * 64);
    float x[U * PV];
#pragma unroll
    for (int u = 0; u < U; ++u) E::unpack(v[u], x + u * PV);
    accumulate<U * PV, EXACT, WANT_Q>(a, x, sc);
  }
  for (int64_t k = nfull * kBatchVecs + tid; k < nvec; k += NTHR) {
    const u32x4 v = load_vec<NT>(vp + k);
    float x[PV];
    E::unpack(v, x);
    accumulate<PV, EXACT, WANT_Q>(a, x, sc);
  }
  {
    const int64_t nscalar = head + (count - tail0);  // < 2*PV <= 16
    if (tid < nscalar) {
      const int64_t idx = (tid < head) ? tid : tail0 + (tid - head);
      float x[1];
      x[0] = E::load1(basep, idx);
      accumulate<1, EXACT, WANT_Q>(a, x, sc);
    }
  }

  // wavefront: common shift, then plain sums
  const float wm = wave_max(a.m);
  rescale(a, wm);
  Part w;
  w.m = wm;
  w.s = wave_sum(a.s);
  w.t = wave_sum(a.t);
  w.q = WANT_Q ? wave_sum(a.q) : 0.f;

  if constexpr (WAVES > 1) {
    __shared__ float sm[WAVES][4];
    if (lane == 0) {
      sm[wave][0] = w.m;
      sm[wave][1] = w.s;
      sm[wave][2] = w.t;
      sm[wave][3] = w.q;
    }
    __syncthreads();
    if (tid == 0) {
      float M = sm[0][0];
#pragma unroll
      for (int i = 1; i < WAVES; ++i) M = __builtin_fmaxf(M, sm[i][0]);
      float S = 0.f, Tt = 0.f, Q = 0.f;
#pragma unroll
      for (int i = 0; i < WAVES; ++i) {
        Part p;
        p.m = sm[i][0];
        p.s = sm[i][1];
        p.t = sm[i][2];
        p.q = sm[i][3];
        rescale(p, M);
        S += p.s;
        Tt += p.t;
        Q += p.q;
      }
      w.m = M;
      w.s = S;
      w.t = Tt;
      w.q = Q;
    }
  }
  return w;
}

template <bool EXACT>
__device__ __forceinline__ Scale<EXACT> make_scale(const float* temperature, int64_t row) {
  Scale<EXACT> sc;
  sc.T = 1.f;
  sc.r = 1.f;
  sc.c = kLog2e;
  if (temperature != nullptr) {
    float T = temperature[row];
    T = (T < kMinTemperature) ? kMinTemperature : T;  // NaN stays NaN, as torch.clamp keeps it
    sc.T = T;
    sc.r = 1.0f / T;
    sc.c = EXACT ? kLog2e : kLog2e / T;
  }
  return sc;
}

// Label logit: one extra element load, issued before the row is streamed.
template <int DT>
__device__ __forceinline__ float load_label_logit(const char* rowp, const int64_t* labels, int64_t row,
                                                  int64_t vocab, bool& label_ok) {
  const int64_t lab = labels[row];
  label_ok = (lab >= 0) && (lab < vocab);
  return label_ok ? Elem<DT>::load1(rowp, lab) : quiet_nan();
}

// One thread turns the row's (M, S, T, Q) into the outputs. The last step is
// done in double: it runs once per row and keeps the result's error at the
// level of the fp32 accumulation.
struct RowResult {
  float lp, H, sps, lse;
};

template <bool EXACT>
__device__ __forceinline__ RowResult row_result(const Part& w, float xl, const Scale<EXACT>& sc) {
  RowResult r;
  if (w.m == neg_inf()) {
    // empty row or every logit -inf: logsumexp = -inf, x - (-inf) and softmax are NaN in torch
    r.lp = quiet_nan();
    r.H = quiet_nan();
    r.sps = quiet_nan();
    r.lse = neg_inf();
  } else if (w.m == pos_inf()) {
    // a +inf logit: logsumexp = +inf
    r.lp = (sc.pre(xl) * sc.c == pos_inf()) ? quiet_nan() : neg_inf();
    r.H = quiet_nan();
    r.sps = quiet_nan();
    r.lse = pos_inf();
  } else {
    const double S = static_cast<double>(w.s);
    const double l2s = log2(S);
    const double yl = static_cast<double>(sc.pre(xl)) * static_cast<double>(sc.c) - static_cast<double>(w.m);
    r.lp = static_cast<float>(kLn2d * (yl - l2s));
    r.H = static_cast<float>(kLn2d * (l2s - static_cast<double>(w.t) / S));
    r.sps = static_cast<float>(static_cast<double>(w.q) / (S * S));
    r.lse = static_cast<float>(kLn2d * (static_cast<double>(w.m) + l2s));
  }
  return r;
}

template <bool EXACT, bool WANT_Q>
__device__ __forceinline__ RowResult finalize_row(const Part& w, float xl, bool label_ok, const Scale<EXACT>& sc,
                                                  int64_t row, float* out_logprob, float* out_entropy,
                                                  float* out_sum_pi_sq, float* out_lse, int32_t* err_flag) {
  RowResult r = row_result<EXACT>(w, xl, sc);
  if (!label_ok) r.lp = quiet_nan();
  if (out_logprob != nullptr) {
    if (!label_ok) atomicOr(err_flag, 1);
    out_logprob[row] = r.lp;
  }
  if (out_entropy != nullptr) out_entropy[row] = r.H;
  if (out_lse != nullptr) out_lse[row] = r.lse;
  if constexpr (WANT_Q) {
    if (out_sum_pi_sq != nullptr) out_sum_pi_sq[row] = r.sps;
  }
  return r;
}

// ---- one workgroup per row ---------------------------------------------------
// grid.x = n_rows, block = WAVES*64 threads; no thread exits early.
template <int DT, int WAVES, int U, bool EXACT, bool NT, bool WANT_Q>
__global__ __launch_bounds__(WAVES * 64) void rowscore_kernel(
    const void* __restrict__ logits, int64_t vocab, int64_t row_stride,
    const int64_t* __restrict__ labels, const float* __restrict__ temperature,
    float* __restrict__ out_logprob, float* __restrict__ out_entropy,
    float* __restrict__ out_sum_pi_sq, float* __restrict__ out_lse, int32_t* err_flag) {
  const int64_t row = blockIdx.x;
  const char* rowp = static_cast<const char*>(logits) + row * row_stride * Elem<DT>::kBytes;
  const Scale<EXACT> sc = make_scale<EXACT>(temperature, row);
  float xl = 0.f;
  bool label_ok = true;
  if (out_logprob != nullptr && threadIdx.x == 0) xl = load_label_logit<DT>(rowp, labels, row, vocab, label_ok);
  const Part w = block_reduce_range<DT, WAVES, U, EXACT, NT, WANT_Q>(rowp, 0, vocab, sc);
  if (threadIdx.x == 0)
    finalize_row<EXACT, WANT_Q>(w, xl, label_ok, sc, row, out_logprob, out_entropy, out_sum_pi_sq, out_lse, err_flag);
}

// ---- packed logits -> padded (B, T_out) response blocks in one launch -----------
// grid.x = n_rows + B, block = WAVES*64.
//   Workgroup r < n_rows scores row r like rowscore_kernel, with the label taken from `labels[r]` or, when
//   `input_ids` is given instead, from the packed ids rolled by one: input_ids[(r + 1) mod n_rows]
//   (verl/workers/engine/fsdp/transformer_impl.py:1177). It finds its sequence b by bisection over cu_seqlens
//   (uniform loads) and, when r lies in that sequence's response window [end - resp - 1, end - 1), also writes its
//   results to column r - (end - resp - 1) of row b of the padded blocks (verl/workers/utils/padding.py:135-138).
//   With no per-token output asked for, a row outside every window is not read at all.
//   Workgroup n_rows + b validates sequence b (offsets inside [0, n_rows] and ordered: VRL_FLAG_SEQ_RANGE; a prompt
//   token before the response and 0 <= resp <= T_out: VRL_FLAG_SLICE_RANGE) and writes the zeros of row b: columns
//   [resp, T_out) of a valid sequence, the whole row of an invalid one, whose rows then write nothing to the blocks.
// Whatever cu_seqlens and response_lens hold, writes stay inside the arrays: block writes go to row b < B, column
// j in [0, T_out). No thread meets a barrier that another one skips: a workgroup leaves as a whole or not at all.
struct ResponseWindow {
  int64_t first;  // first row of the window
  int64_t resp;   // its length
  bool ok;
};

__device__ __forceinline__ ResponseWindow response_window(const int64_t* cu_seqlens, const int64_t* response_lens,
                                                          int64_t b, int64_t B, int64_t n_rows, int64_t T_out,
                                                          int* why) {
  const int64_t begin = cu_seqlens[b];
  const int64_t end = cu_seqlens[b + 1];
  const int64_t resp = response_lens[b];
  const bool span_ok = (begin >= 0) && (end <= n_rows) && (end >= begin) && (b != 0 || begin == 0) &&
                       (b + 1 != B || end == n_rows);
  ResponseWindow w;
  w.resp = resp;
  w.first = 0;
  bool resp_ok = false;
  if (span_ok && resp >= 0 && resp <= T_out) {  // only now is end - resp - 1 known not to wrap
    w.first = end - resp - 1;
    resp_ok = w.first >= begin;
  }
  w.ok = span_ok && resp_ok;
  *why = span_ok ? (resp_ok ? 0 : 2) : 4;
  return w;
}

template <int DT, int WAVES, int U, bool EXACT>
__global__ __launch_bounds__(WAVES * 64) void score_responses_kernel(
    const void* __restrict__ logits, int64_t n_rows, int64_t vocab, int64_t row_stride,
    const int64_t* __restrict__ labels, const int64_t* __restrict__ input_ids,
    const float* __restrict__ temperature, const int64_t* __restrict__ cu_seqlens,
    const int64_t* __restrict__ response_lens, int64_t B, int64_t T_out, float* __restrict__ out_logprob,
    float* __restrict__ out_entropy, float* __restrict__ resp_logprob, float* __restrict__ resp_entropy,
    float* __restrict__ resp_lse, int32_t* err_flag) {
  constexpr int NTHR = WAVES * 64;
  const int64_t wg = blockIdx.x;
  if (wg >= n_rows) {
    // sequence workgroup: validation and the zeros of row b
    const int64_t b = wg - n_rows;
    int why = 0;
    const ResponseWindow w = response_window(cu_seqlens, response_lens, b, B, n_rows, T_out, &why);
    if (why != 0 && threadIdx.x == 0) atomicOr(err_flag, why);
    const int64_t from = w.ok ? w.resp : 0;
    for (int64_t j = from + threadIdx.x; j < T_out; j += NTHR) {
      if (resp_logprob != nullptr) resp_logprob[b * T_out + j] = 0.f;
      if (resp_entropy != nullptr) resp_entropy[b * T_out + j] = 0.f;
      if (resp_lse != nullptr) resp_lse[b * T_out + j] = 0.f;
    }
    return;
  }
  const int64_t row = wg;
  // sequence of this row: the largest b with cu[b] <= row (bisection; uniform over the workgroup)
  int64_t lo = 0, hi = B;  // invariant: answer in [lo, hi)
  while (hi - lo > 1) {
    const int64_t mid = (lo + hi) >> 1;
    if (cu_seqlens[mid] <= row) lo = mid; else hi = mid;
  }
  bool in_window = false;
  int64_t col = 0;
  const int64_t b = lo;
  if (B > 0 && cu_seqlens[b] <= row && row < cu_seqlens[b + 1]) {
    int why = 0;
    const ResponseWindow w = response_window(cu_seqlens, response_lens, b, B, n_rows, T_out, &why);
    if (w.ok) {
      col = row - w.first;
      in_window = col >= 0 && col < w.resp;
    }
  }
  const bool per_token = (out_logprob != nullptr) || (out_entropy != nullptr);
  if (!per_token && !in_window) return;  // the whole workgroup: this row's logits are never read

  const char* rowp = static_cast<const char*>(logits) + row * row_stride * Elem<DT>::kBytes;
  const Scale<EXACT> sc = make_scale<EXACT>(temperature, row);
  const bool want_lp = (out_logprob != nullptr) || (resp_logprob != nullptr);
  float xl = 0.f;
  bool label_ok = true;
  if (want_lp && threadIdx.x == 0) {
    int64_t lab;
    if (input_ids != nullptr) {
      lab = input_ids[row + 1 < n_rows ? row + 1 : 0];
    } else {
      lab = labels[row];
    }
    label_ok = (lab >= 0) && (lab < vocab);
    xl = label_ok ? Elem<DT>::load1(rowp, lab) : quiet_nan();
  }
  const Part w = block_reduce_range<DT, WAVES, U, EXACT, true, false>(rowp, 0, vocab, sc);
  if (threadIdx.x == 0) {
    if (want_lp && !label_ok && out_logprob == nullptr) atomicOr(err_flag, 1);  // finalize_row flags it otherwise
    const RowResult r = finalize_row<EXACT, false>(w, xl, label_ok, sc, row, out_logprob, out_entropy, nullptr,
                                                   nullptr, err_flag);
    if (in_window) {
      if (resp_logprob != nullptr) resp_logprob[b * T_out + col] = r.lp;
      if (resp_entropy != nullptr) resp_entropy[b * T_out + col] = r.H;
      if (resp_lse != nullptr) resp_lse[b * T_out + col] = r.lse;
    }
  }
}

// ---- few rows: several workgroups per row ------------------------------------
// grid.x = n_rows * n_splits. Workgroup (row, k) reduces elements
// [k*slice, min((k+1)*slice, vocab)) and stores its partial (M, S, T, Q) at
// partials[(row*n_splits + k)*4 ...]; rowscore_merge_kernel finishes the rows.
template <int DT, int WAVES, int U, bool EXACT, bool NT, bool WANT_Q>
__global__ __launch_bounds__(WAVES * 64) void rowscore_split_kernel(
    const void* __restrict__ logits, int64_t vocab, int64_t row_stride,
    const float* __restrict__ temperature, int n_splits, int64_t slice, float* __restrict__ partials) {
  const int64_t row = blockIdx.x / n_splits;
  const int k = static_cast<int>(blockIdx.x % n_splits);
  const char* rowp = static_cast<const char*>(logits) + row * row_stride * Elem<DT>::kBytes;
  const Scale<EXACT> sc = make_scale<EXACT>(temperature, row);
  int64_t lo = k * slice;
  int64_t hi = lo + slice;
  if (lo > vocab) lo = vocab;
  if (hi > vocab) hi = vocab;
  const Part w = block_reduce_range<DT, WAVES, U, EXACT, NT, WANT_Q>(rowp, lo, hi, sc);
  if (threadIdx.x == 0) {
    float* dst = partials + (row * n_splits + k) * 4;
    dst[0] = w.m;
    dst[1] = w.s;
    dst[2] = w.t;
    dst[3] = w.q;
  }
}

// grid.x = ceil(n_rows / 64), block = 64: one lane per row merges that row's
// n_splits partials in index order (deterministic) and writes the outputs.
template <int DT, bool EXACT, bool WANT_Q>
__global__ __launch_bounds__(64) void rowscore_merge_kernel(
    const void* __restrict__ logits, int64_t n_rows, int64_t vocab, int64_t row_stride,
    const int64_t* __restrict__ labels, const float* __restrict__ temperature, int n_splits,
    const float* __restrict__ partials, float* __restrict__ out_logprob, float* __restrict__ out_entropy,
    float* __restrict__ out_sum_pi_sq, float* __restrict__ out_lse, int32_t* err_flag) {
  const int64_t row = static_cast<int64_t>(blockIdx.x) * 64 + threadIdx.x;
  if (row >= n_rows) return;
  const char* rowp = static_cast<const char*>(logits) + row * row_stride * Elem<DT>::kBytes;
  const Scale<EXACT> sc = make_scale<EXACT>(temperature, row);
  float xl = 0.f;
  bool label_ok = true;
  if (out_logprob != nullptr) xl = load_label_logit<DT>(rowp, labels, row, vocab, label_ok);
  const float* src = partials + row * n_splits * 4;
  float M = src[0];
  for (int k = 1; k < n_splits; ++k) M = __builtin_fmaxf(M, src[k * 4]);
  Part w;
  w.m = M;
  w.s = 0.f;
  w.t = 0.f;
  w.q = 0.f;
  for (int k = 0; k < n_splits; ++k) {
    Part p;
    p.m = src[k * 4 + 0];
    p.s = src[k * 4 + 1];
    p.t = src[k * 4 + 2];
    p.q = src[k * 4 + 3];
    rescale(p, M);
    w.s += p.s;
    w.t += p.t;
    w.q += p.q;
  }
  finalize_row<EXACT, WANT_Q>(w, xl, label_ok, sc, row, out_logprob, out_entropy, out_sum_pi_sq, out_lse, err_flag);
}

// ---- label log-prob from a known logsumexp ------------------------------------
// grid.x = ceil(n_rows / 256), block = 256: one lane per row, no barrier. logprob = z[label] - lse with the same
// scaling of the label logit as finalize_row (double, one rounding at the end); lse = -inf / +inf / NaN propagate by
// plain arithmetic to what torch's `x.gather(label) - logsumexp(x)` gives.
template <int DT, bool EXACT>
__global__ __launch_bounds__(256) void label_logprob_kernel(
    const void* __restrict__ logits, int64_t n_rows, int64_t vocab, int64_t row_stride,
    const int64_t* __restrict__ labels, const float* __restrict__ temperature, const float* __restrict__ lse,
    float* __restrict__ out_logprob, int32_t* err_flag) {
  const int64_t row = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  if (row >= n_rows) return;
  const char* rowp = static_cast<const char*>(logits) + row * row_stride * Elem<DT>::kBytes;
  const Scale<EXACT> sc = make_scale<EXACT>(temperature, row);
  bool label_ok = true;
  const float xl = load_label_logit<DT>(rowp, labels, row, vocab, label_ok);
  float lp = quiet_nan();
  if (label_ok) {
    const double z = kLn2d * (static_cast<double>(sc.pre(xl)) * static_cast<double>(sc.c));
    lp = static_cast<float>(z - static_cast<double>(lse[row]));
  } else {
    atomicOr(err_flag, 1);
  }
  out_logprob[row] = lp;
}

}  // namespace vrl
