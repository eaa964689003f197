// Rollout correction on (B, T) log-probs in one launch: importance-sampling weights (token or sequence
// level, truncated or IcePop-zeroed), the rejection mask of any combination of the eleven k1/k2/k3
// criteria, and per-sequence partial sums from which every metric of the step is derived on the host.
//
// One workgroup per sequence, two passes over its tokens (they stay in cache):
//   pass 1 reduces the per-token statistics of the clamped log ratio
//          k1 = -lr, k2 = lr^2 / 2, k3 = exp(lr) - 1 - lr,  lr = clamp(old - rollout, +-20)
//          to the sequence's sums / means / maxima, which decide the sequence-level criteria and
//          the sequence-level weight exp(clamp(sum lr, +-20));
//   pass 2 writes weight and keep flag per token and reduces what depends on them.
// All reductions run in a fixed order (DPP inside a wavefront, LDS across), so results are deterministic.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "rowscore_kernels.h"

namespace vrl {

constexpr float kSafetyBound = 20.0f;  // verl/trainer/ppo/rollout_corr_helper.py:75
constexpr int kNumRsOptions = 11;

// order of the options everywhere: bits of CorrCfg::rs_bits and of seq_keep_bits
enum RsOption {
  kTokenK1 = 0, kTokenK2, kTokenK3, kSeqSumK1, kSeqSumK2, kSeqSumK3, kSeqMeanK1, kSeqMeanK2, kSeqMeanK3,
  kSeqMaxK2, kSeqMaxK3
};

// per-sequence statistics, one float each
enum CorrStat {
  kN = 0, kSumOld, kSumRoll, kSumLr, kSumK3Raw, kSumRho2, kSumK1, kSumK2, kSumK3,
  kMaxK1, kMinK1, kMaxK2, kMinK2, kMaxK3, kMinK3,
  kTokHi0, kTokLo0, kTokCl0, kTokCl20,  // token_k1: count above upper, count below lower, sum clamp, sum clamp^2
  kTokHi1, kTokLo1, kTokCl1, kTokCl21,  // token_k2
  kTokHi2, kTokLo2, kTokCl2, kTokCl22,  // token_k3
  kTokMasked0, kTokMasked1, kTokMasked2,
  kFinalMasked,
  kSumW, kSumWRaw, kMaxW, kMinW, kCntRawHi, kCntRawLo, kSumWc, kSumWc2, kCntOob,
  kNumCorrStats
};

struct CorrCfg {
  int is_mode;            // 0 off, 1 token, 2 sequence
  int icepop;             // 0: clamp to is_upper, 1: zero outside [is_lower, is_upper]
  float is_upper;
  float is_lower;         // IcePop lower bound
  float is_lower_metric;  // lower bound of the "fraction_low" diagnostics (1/upper unless IcePop)
  uint32_t rs_bits;
  float rs_lo[kNumRsOptions];  // compared as is (log of the ratio bound for k1 options)
  float rs_hi[kNumRsOptions];
};

enum ReduceKind { kRedSum = 0, kRedMax = 1, kRedMin = 2 };

// Reduce `count` per-thread values over the workgroup; every thread gets every result.
template <int WAVES, int MAXN, int COUNT>
__device__ __forceinline__ void block_reduce_many(float* vals, const uint8_t* kinds, float (*sm)[MAXN],
                                                  float* out_sm) {
  static_assert(COUNT <= MAXN && COUNT <= WAVES * 64, "too many values for one reduction round");
  constexpr int count = COUNT;
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
#pragma unroll
  for (int i = 0; i < count; ++i) {
    float v = vals[i];
    if (kinds[i] == kRedSum) {
      v = wave_sum(v);
    } else if (kinds[i] == kRedMax) {
      v = wave_max(v);
    } else {
      v = -wave_max(-v);
    }
    if (lane == 0) sm[wave][i] = v;
  }
  __syncthreads();
  if (static_cast<int>(threadIdx.x) < count) {
    const int i = threadIdx.x;
    float r = sm[0][i];
    for (int w = 1; w < WAVES; ++w) {
      const float o = sm[w][i];
      r = (kinds[i] == kRedSum) ? r + o : ((kinds[i] == kRedMax) ? __builtin_fmaxf(r, o) : __builtin_fminf(r, o));
    }
    out_sm[i] = r;
  }
  __syncthreads();
#pragma unroll
  for (int i = 0; i < count; ++i) vals[i] = out_sm[i];
  __syncthreads();
}

__device__ __forceinline__ float clampf(float x, float lo, float hi) {
  return __builtin_fminf(__builtin_fmaxf(x, lo), hi);
}

// grid.x = B, block = WAVES*64. mask may be NULL (all valid). weights / keep may be NULL.
template <int WAVES>
__global__ __launch_bounds__(WAVES * 64) void rollout_corr_kernel(
    const float* __restrict__ old_lp, const float* __restrict__ roll_lp, const uint8_t* __restrict__ mask,
    int64_t T, const CorrCfg cfg, float* __restrict__ weights, uint8_t* __restrict__ keep,
    float* __restrict__ stats, int32_t* __restrict__ seq_keep_bits) {
  constexpr int NTHR = WAVES * 64;
  constexpr int MAXN = 32;
  __shared__ float sm[WAVES][MAXN];
  __shared__ float out_sm[MAXN];
  const int tid = threadIdx.x;
  const int64_t b = blockIdx.x;
  const float* po = old_lp + b * T;
  const float* pr = roll_lp + b * T;
  const uint8_t* pm = (mask != nullptr) ? mask + b * T : nullptr;
  const float inf = pos_inf();

  const bool tok_on[3] = {(cfg.rs_bits >> kTokenK1 & 1u) != 0, (cfg.rs_bits >> kTokenK2 & 1u) != 0,
                          (cfg.rs_bits >> kTokenK3 & 1u) != 0};

  // ---- pass 1 ----
  enum { P_N, P_OLD, P_ROLL, P_LR, P_K3RAW, P_RHO2, P_K1, P_K2, P_K3, P_MAXK1, P_MINK1, P_MAXK2, P_MINK2, P_MAXK3,
         P_MINK3, P_HI0, P_LO0, P_CL0, P_CL20, P_HI1, P_LO1, P_CL1, P_CL21, P_HI2, P_LO2, P_CL2, P_CL22, P1_COUNT };
  float a[P1_COUNT];
  uint8_t kinds[P1_COUNT];
  for (int i = 0; i < P1_COUNT; ++i) {
    a[i] = 0.f;
    kinds[i] = kRedSum;
  }
  a[P_MAXK1] = a[P_MAXK2] = a[P_MAXK3] = -inf;
  a[P_MINK1] = a[P_MINK2] = a[P_MINK3] = inf;
  kinds[P_MAXK1] = kinds[P_MAXK2] = kinds[P_MAXK3] = kRedMax;
  kinds[P_MINK1] = kinds[P_MINK2] = kinds[P_MINK3] = kRedMin;

  for (int64_t i = tid; i < T; i += NTHR) {
    const bool valid = (pm != nullptr) ? (pm[i] != 0) : true;
    if (!valid) continue;
    const float o = po[i], r = pr[i];
    const float lr_raw = o - r;
    const float lr = clampf(lr_raw, -kSafetyBound, kSafetyBound);
    const float k1 = -lr;
    const float k2 = 0.5f * (lr * lr);
    const float ex = expf(lr);
    const float k3 = ex - 1.0f - lr;
    a[P_N] += 1.f;
    a[P_OLD] += o;
    a[P_ROLL] += r;
    a[P_LR] += lr_raw;
    a[P_K3RAW] += expf(lr_raw) - lr_raw - 1.0f;
    a[P_RHO2] += ex * ex;
    a[P_K1] += k1;
    a[P_K2] += k2;
    a[P_K3] += k3;
    a[P_MAXK1] = __builtin_fmaxf(a[P_MAXK1], k1);
    a[P_MINK1] = __builtin_fminf(a[P_MINK1], k1);
    a[P_MAXK2] = __builtin_fmaxf(a[P_MAXK2], k2);
    a[P_MINK2] = __builtin_fminf(a[P_MINK2], k2);
    a[P_MAXK3] = __builtin_fmaxf(a[P_MAXK3], k3);
    a[P_MINK3] = __builtin_fminf(a[P_MINK3], k3);
    const float ks[3] = {k1, k2, k3};
#pragma unroll
    for (int j = 0; j < 3; ++j) {
      if (!tok_on[j]) continue;
      const float hi = cfg.rs_hi[j];
      const float lo = (j == 0) ? cfg.rs_lo[0] : 0.f;  // k1 has a lower bound, k2/k3 clamp at 0
      const float c = clampf(ks[j], lo, hi);
      a[P_HI0 + 4 * j] += (ks[j] > hi) ? 1.f : 0.f;
      if (j == 0) a[P_LO0] += (ks[j] < lo) ? 1.f : 0.f;
      a[P_CL0 + 4 * j] += c;
      a[P_CL20 + 4 * j] += c * c;
    }
  }
  block_reduce_many<WAVES, MAXN, P1_COUNT>(a, kinds, sm, out_sm);

  // ---- sequence-level decisions (every thread computes the same) ----
  const float n = a[P_N];
  const float denom = n + 1e-8f;  // masked_mean divides by mask.sum() + 1e-8
  const float ssum[3] = {a[P_K1], a[P_K2], a[P_K3]};
  const float smean[3] = {a[P_K1] / denom, a[P_K2] / denom, a[P_K3] / denom};
  const float smax[3] = {n > 0.f ? a[P_MAXK1] : 0.f, n > 0.f ? a[P_MAXK2] : 0.f, n > 0.f ? a[P_MAXK3] : 0.f};
  uint32_t seq_bits = 0;   // bit set = the sequence PASSES that (enabled) sequence-level criterion
  bool seq_keep = true;
  for (int opt = kSeqSumK1; opt < kNumRsOptions; ++opt) {
    if (((cfg.rs_bits >> opt) & 1u) == 0) continue;
    float s;
    bool is_k1 = false;
    if (opt <= kSeqSumK3) {
      s = ssum[opt - kSeqSumK1];
      is_k1 = (opt == kSeqSumK1);
    } else if (opt <= kSeqMeanK3) {
      s = smean[opt - kSeqMeanK1];
      is_k1 = (opt == kSeqMeanK1);
    } else {
      s = smax[opt - kSeqMaxK2 + 1];
    }
    const bool pass = is_k1 ? (s >= cfg.rs_lo[opt] && s <= cfg.rs_hi[opt]) : (s <= cfg.rs_hi[opt]);
    if (pass) seq_bits |= (1u << opt);
    seq_keep = seq_keep && pass;
  }
  const float seq_raw_w = expf(clampf(a[P_LR], -kSafetyBound, kSafetyBound));

  // ---- pass 2 ----
  enum { Q_MASK0, Q_MASK1, Q_MASK2, Q_FINAL, Q_W, Q_WRAW, Q_MAXW, Q_MINW, Q_RAWHI, Q_RAWLO, Q_WC, Q_WC2, Q_OOB, P2_COUNT };
  float q[P2_COUNT];
  uint8_t kinds2[P2_COUNT];
  for (int i = 0; i < P2_COUNT; ++i) {
    q[i] = 0.f;
    kinds2[i] = kRedSum;
  }
  q[Q_MAXW] = -inf;
  q[Q_MINW] = inf;
  kinds2[Q_MAXW] = kRedMax;
  kinds2[Q_MINW] = kRedMin;

  for (int64_t i = tid; i < T; i += NTHR) {
    const bool valid = (pm != nullptr) ? (pm[i] != 0) : true;
    const float lr = clampf(po[i] - pr[i], -kSafetyBound, kSafetyBound);
    const float ex = expf(lr);
    const float ks[3] = {-lr, 0.5f * (lr * lr), ex - 1.0f - lr};
    bool k = seq_keep;
#pragma unroll
    for (int j = 0; j < 3; ++j) {
      if (!tok_on[j]) continue;
      const bool pass = (j == 0) ? (ks[0] >= cfg.rs_lo[0] && ks[0] <= cfg.rs_hi[0]) : (ks[j] <= cfg.rs_hi[j]);
      if (valid && !pass) q[Q_MASK0 + j] += 1.f;
      k = k && pass;
    }
    if (keep != nullptr) keep[b * T + i] = static_cast<uint8_t>(k);
    if (valid && !k) q[Q_FINAL] += 1.f;
    if (cfg.is_mode != 0) {
      const float m = valid ? 1.f : 0.f;
      const float raw = ((cfg.is_mode == 1) ? ex : seq_raw_w) * m;
      float w;
      if (cfg.icepop) {
        w = (raw >= cfg.is_lower && raw <= cfg.is_upper) ? raw : 0.f;
      } else {
        w = __builtin_fminf(raw, cfg.is_upper);
      }
      if (weights != nullptr) weights[b * T + i] = w;
      if (valid) {
        const float wc = clampf(w, 0.f, cfg.is_upper);
        q[Q_W] += w;
        q[Q_WRAW] += raw;
        q[Q_MAXW] = __builtin_fmaxf(q[Q_MAXW], w);
        q[Q_MINW] = __builtin_fminf(q[Q_MINW], w);
        q[Q_RAWHI] += (raw > cfg.is_upper) ? 1.f : 0.f;
        q[Q_RAWLO] += (raw < cfg.is_lower_metric) ? 1.f : 0.f;
        q[Q_WC] += wc;
        q[Q_WC2] += wc * wc;
        q[Q_OOB] += (cfg.icepop && (raw < cfg.is_lower || raw > cfg.is_upper)) ? 1.f : 0.f;
      }
    }
  }
  block_reduce_many<WAVES, MAXN, P2_COUNT>(q, kinds2, sm, out_sm);

  if (tid == 0) {
    float* s = stats + b * kNumCorrStats;
    s[kN] = a[P_N];
    s[kSumOld] = a[P_OLD];
    s[kSumRoll] = a[P_ROLL];
    s[kSumLr] = a[P_LR];
    s[kSumK3Raw] = a[P_K3RAW];
    s[kSumRho2] = a[P_RHO2];
    s[kSumK1] = a[P_K1];
    s[kSumK2] = a[P_K2];
    s[kSumK3] = a[P_K3];
    s[kMaxK1] = a[P_MAXK1];
    s[kMinK1] = a[P_MINK1];
    s[kMaxK2] = a[P_MAXK2];
    s[kMinK2] = a[P_MINK2];
    s[kMaxK3] = a[P_MAXK3];
    s[kMinK3] = a[P_MINK3];
    for (int j = 0; j < 12; ++j) s[kTokHi0 + j] = a[P_HI0 + j];
    s[kTokMasked0] = q[Q_MASK0];
    s[kTokMasked1] = q[Q_MASK1];
    s[kTokMasked2] = q[Q_MASK2];
    s[kFinalMasked] = q[Q_FINAL];
    s[kSumW] = q[Q_W];
    s[kSumWRaw] = q[Q_WRAW];
    s[kMaxW] = q[Q_MAXW];
    s[kMinW] = q[Q_MINW];
    s[kCntRawHi] = q[Q_RAWHI];
    s[kCntRawLo] = q[Q_RAWLO];
    s[kSumWc] = q[Q_WC];
    s[kSumWc2] = q[Q_WC2];
    s[kCntOob] = q[Q_OOB];
    seq_keep_bits[b] = static_cast<int32_t>(seq_bits);
  }
}

}  // namespace vrl
