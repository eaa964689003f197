/*
 * TEST INFRASTRUCTURE — plain-C restatement of the scoring path and of the
 * SPEC-RL verify rule, independent of torch. Only tests/, smoke() and the
 * cpu_baseline leg of bench.py may use it; the product never links it.
 *
 * Scoring follows the textbook two-pass form of what the reference computes
 *   verl/utils/torch_functional.py:194-198  logprob = x[label] - logsumexp(x)
 *   verl/utils/torch_functional.py:243-244  entropy = logsumexp(x) - sum(softmax(x) * x)
 *   verl/workers/engine/fsdp/transformer_impl.py:1357  x = logits / max(T, 1e-8), rounded to fp32
 * with every reduction in double, so it serves as ground truth for both the
 * torch restatement (oracle/scoring.py) and the HIP kernel.
 * As in torch, a -inf logit makes the entropy NaN (0 * -inf) and leaves the
 * log-prob defined; a row of only -inf gives NaN for both.
 *
 * Verify follows oracle/verify.py (decisions D1-D6 there); all token
 * arithmetic is single fp32 operations, compiled with -ffp-contract=off.
 */
#include <math.h>
#include <stdint.h>
#include <string.h>

static float bf16_to_f32(uint16_t h) {
  uint32_t u = ((uint32_t)h) << 16;
  float f;
  memcpy(&f, &u, sizeof f);
  return f;
}

static float load_elem(const void* base, int dtype, int64_t idx) {
  if (dtype == 0) return ((const float*)base)[idx];
  return bf16_to_f32(((const uint16_t*)base)[idx]);
}

/* dtype: 0 = fp32, 1 = bf16. labels may be NULL (then out_logprob is not written). */
int vrl_oracle_rowscore(const void* logits, int dtype, int64_t n_rows, int64_t vocab, int64_t row_stride,
                        const int64_t* labels, const float* temperature, double* out_logprob,
                        double* out_entropy) {
  if (dtype != 0 && dtype != 1) return -2;
  if (n_rows < 0 || vocab <= 0 || row_stride < vocab) return -3;
  int64_t r;
#pragma omp parallel for schedule(static)
  for (r = 0; r < n_rows; ++r) {
    const int64_t base = r * row_stride;
    float T = 1.0f;
    int scaled = 0;
    if (temperature) {
      T = temperature[r];
      if (T < 1e-8f) T = 1e-8f;
      scaled = 1;
    }
    double mx = -INFINITY;
    int has_nan = 0;
    for (int64_t v = 0; v < vocab; ++v) {
      float x = load_elem(logits, dtype, base + v);
      if (scaled) x = x / T; /* fp32 quotient, as the reference forms it */
      if (x != x) has_nan = 1;
      if ((double)x > mx) mx = (double)x;
    }
    double s = 0.0, t = 0.0;
    if (isfinite(mx)) {
      for (int64_t v = 0; v < vocab; ++v) {
        float x = load_elem(logits, dtype, base + v);
        if (scaled) x = x / T;
        const double e = exp((double)x - mx);
        s += e;
        t += e * (double)x; /* 0 * -inf = NaN, like torch */
      }
    }
    double lse, H;
    if (has_nan) {
      lse = NAN;
      H = NAN;
    } else if (mx == -INFINITY) {
      lse = -INFINITY;
      H = NAN;
    } else if (mx == INFINITY) {
      lse = INFINITY;
      H = NAN;
    } else {
      lse = mx + log(s);
      H = lse - t / s;
    }
    if (out_entropy) out_entropy[r] = H;
    if (out_logprob && labels) {
      const int64_t lab = labels[r];
      if (lab < 0 || lab >= vocab) {
        out_logprob[r] = NAN;
      } else {
        float xl = load_elem(logits, dtype, base + lab);
        if (scaled) xl = xl / T;
        out_logprob[r] = (double)xl - lse; /* -inf - -inf and inf - inf are NaN, like torch */
      }
    }
  }
  return 0;
}

/* Sequence b owns tokens [cu[b], cu[b+1]) if cu != NULL, else [b*T, (b+1)*T). */
int vrl_oracle_spec_verify(const float* logp_new, const float* logp_old, const float* log_u,
                           const uint8_t* mask, const int64_t* cu, int64_t B, int64_t T,
                           float thresh_offset, float near_eps, uint8_t* accept, int32_t* first_reject,
                           int32_t* prefix_len, int32_t* near_count, const int64_t* draft_ids,
                           int64_t pad_id, int64_t* out_ids, uint8_t* out_mask) {
  if (B < 0 || T < 0) return -3;
  for (int64_t b = 0; b < B; ++b) {
    const int64_t start = cu ? cu[b] : b * T;
    int64_t len = cu ? cu[b + 1] - cu[b] : T;
    if (len < 0) len = 0;
    int64_t first = -1, last_valid = 0;
    int32_t near = 0;
    for (int64_t i = 0; i < len; ++i) {
      const int64_t g = start + i;
      const int valid = mask ? (mask[g] != 0) : 1;
      const float d = logp_new[g] - logp_old[g];
      const float tau = log_u[g] + thresh_offset;
      const int ok = d >= tau;
      accept[g] = (uint8_t)(valid && ok);
      if (valid) {
        last_valid = i + 1;
        if (!ok && first < 0) first = i;
        if (fabsf(d - tau) < near_eps) ++near;
      }
    }
    const int64_t f = first < 0 ? last_valid : first;
    int32_t cnt = 0;
    for (int64_t i = 0; i < f; ++i) cnt += mask ? (mask[start + i] != 0) : 1;
    first_reject[b] = (int32_t)f;
    prefix_len[b] = cnt;
    near_count[b] = near;
    if (draft_ids && out_ids && out_mask) {
      for (int64_t i = 0; i < len; ++i) {
        const int64_t g = start + i;
        const int keep = i < f;
        out_ids[g] = keep ? draft_ids[g] : pad_id;
        out_mask[g] = keep ? (uint8_t)(mask ? (mask[g] != 0) : 1) : (uint8_t)0;
      }
    }
  }
  return 0;
}
