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
//
// Mapping. One workgroup of WAVES wavefronts owns one row. A register batch is
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
};

// Bring p to the shift M >= p.m. A partial that has seen nothing finite
// (m == -inf, s == 0) stays zero instead of producing 0*inf.
__device__ __forceinline__ void rescale(Part& p, float M) {
  const bool dead = (p.m == neg_inf());
  const float dm = dead ? 0.f : p.m - M;
  const float alpha = dead ? 0.f : hw_exp2(dm);
  p.t = alpha * (p.t + dm * p.s);
  p.s = alpha * p.s;
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
template <int N, bool EXACT>
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
  float ps = 0.f, pt = 0.f;
#pragma unroll
  for (int i = 0; i < N; ++i) {
    const float d = __builtin_fmaf(x[i], sc.c, -sub);
    const float e = hw_exp2(d);
    ps += e;
    pt = __builtin_fmaf(e, d, pt);
  }
  a.s += ps;
  a.t += pt;
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

// ---- the kernel ------------------------------------------------------------
// grid.x = n_rows, block = WAVES*64 threads. All threads of a block reach the
// reductions and the barrier (no early exit), so EXEC is full for the DPP ops.
template <int DT, int WAVES, int U, bool EXACT, bool NT>
__global__ __launch_bounds__(WAVES * 64) void rowscore_kernel(
    const void* __restrict__ logits, int64_t vocab, int64_t row_stride,
    const int64_t* __restrict__ labels, const float* __restrict__ temperature,
    float* __restrict__ out_logprob, float* __restrict__ out_entropy, int32_t* err_flag) {
  using E = Elem<DT>;
  constexpr int NTHR = WAVES * 64;
  constexpr int PV = E::kPerVec;
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int64_t row = blockIdx.x;
  const char* rowp = static_cast<const char*>(logits) + row * row_stride * E::kBytes;

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

  // Label logit: one extra element load by thread 0, issued before the stream.
  float xl = 0.f;
  bool label_ok = true;
  if (out_logprob != nullptr && tid == 0) {
    const int64_t lab = labels[row];
    label_ok = (lab >= 0) && (lab < vocab);
    xl = label_ok ? E::load1(rowp, lab) : quiet_nan();
  }

  // Split the row into [head scalars][16-byte vectors][tail scalars].
  const uintptr_t addr = reinterpret_cast<uintptr_t>(rowp);
  int64_t head = static_cast<int64_t>(((16u - (addr & 15u)) & 15u) / E::kBytes);
  if (head > vocab) head = vocab;
  const int64_t nvec = (vocab - head) / PV;
  const int64_t tail0 = head + nvec * PV;
  const u32x4* vp = reinterpret_cast<const u32x4*>(rowp + head * E::kBytes);

  Part a;
  a.m = neg_inf();
  a.s = 0.f;
  a.t = 0.f;

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
    accumulate<U * PV, EXACT>(a, x, sc);
  }
  for (int64_t k = nfull * kBatchVecs + tid; k < nvec; k += NTHR) {
    const u32x4 v = load_vec<NT>(vp + k);
    float x[PV];
    E::unpack(v, x);
    accumulate<PV, EXACT>(a, x, sc);
  }
  {
    const int64_t nscalar = head + (vocab - tail0);  // < 2*PV <= 16
    if (tid < nscalar) {
      const int64_t idx = (tid < head) ? tid : tail0 + (tid - head);
      float x[1];
      x[0] = E::load1(rowp, idx);
      accumulate<1, EXACT>(a, x, sc);
    }
  }

  // wavefront: common shift, then plain sums
  const float wm = wave_max(a.m);
  rescale(a, wm);
  Part w;
  w.m = wm;
  w.s = wave_sum(a.s);
  w.t = wave_sum(a.t);

  if constexpr (WAVES > 1) {
    __shared__ float sm[WAVES][3];
    if (lane == 0) {
      sm[wave][0] = w.m;
      sm[wave][1] = w.s;
      sm[wave][2] = w.t;
    }
    __syncthreads();
    if (tid == 0) {
      float M = sm[0][0];
#pragma unroll
      for (int i = 1; i < WAVES; ++i) M = __builtin_fmaxf(M, sm[i][0]);
      float S = 0.f, Tt = 0.f;
#pragma unroll
      for (int i = 0; i < WAVES; ++i) {
        Part p;
        p.m = sm[i][0];
        p.s = sm[i][1];
        p.t = sm[i][2];
        rescale(p, M);
        S += p.s;
        Tt += p.t;
      }
      w.m = M;
      w.s = S;
      w.t = Tt;
    }
  }

  if (tid == 0) {
    float lp, H;
    if (w.m == neg_inf()) {
      // empty row or every logit -inf: logsumexp = -inf, x - (-inf) and softmax are NaN in torch
      lp = quiet_nan();
      H = quiet_nan();
    } else if (w.m == pos_inf()) {
      // a +inf logit: logsumexp = +inf
      lp = (sc.pre(xl) * sc.c == pos_inf()) ? quiet_nan() : neg_inf();
      H = quiet_nan();
    } else {
      const double S = static_cast<double>(w.s);
      const double l2s = log2(S);
      const double yl = static_cast<double>(sc.pre(xl)) * static_cast<double>(sc.c) - static_cast<double>(w.m);
      lp = static_cast<float>(kLn2d * (yl - l2s));
      H = static_cast<float>(kLn2d * (l2s - static_cast<double>(w.t) / S));
    }
    if (out_logprob != nullptr) {
      if (!label_ok) {
        lp = quiet_nan();
        atomicOr(err_flag, 1);
      }
      out_logprob[row] = lp;
    }
    if (out_entropy != nullptr) out_entropy[row] = H;
  }
}

}  // namespace vrl
