// Backward of the row op: one read of the logits, one write of their gradient.
//
// With z = x / T, p = softmax(z), log p_v = z_v - lse, H the row's entropy and
// (g_l, g_h) the incoming gradients of the label log-prob and of the entropy,
//   d/dz_v = g_l * (1[v == label] - p_v) - g_h * p_v * (log p_v + H)
//   d/dx_v = (d/dz_v) / T
// which is the closed form the reference states at
// verl/utils/experimental/torch_functional.py:66-79. In the log2 domain:
//   u = fma(x, c, -lse*log2e);  p = v_exp_f32(u);  dx = p * fma(u, a, b)  (+ g_l/T at the label)
// with a = -g_h*ln2/T and b = -(g_l + g_h*H)/T constant over the row.
// For fp32 logits the exponent is formed the way torch forms it instead, so that its only rounding of size
// ulp(|z|) is the one torch has too: z = RN(x / T) (exact division, as in the forward kernel), d = z - lse
// (= log p), p = v_exp_f32(d * log2e), dx = p * fma(d, a', b) with a' = -g_h / T. With peaked rows at low
// temperature (|z| ~ 100) the folded form above is ~5x further from the fp64 gradient than torch's fp32 autograd.
// lse and H come from the forward pass. The gradient has the logits' dtype and
// may be written over the logits themselves (every element is read and then
// written by the same lane).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <type_traits>

#include "rowscore_kernels.h"

namespace vrl {

typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));

constexpr float kLn2f = 0.69314718055994530942f;

template <int DT>
struct ElemOut;

template <>
struct ElemOut<0> {
  __device__ static __forceinline__ u32x4 pack(const float* y) {
    u32x4 v;
    v.x = __float_as_uint(y[0]);
    v.y = __float_as_uint(y[1]);
    v.z = __float_as_uint(y[2]);
    v.w = __float_as_uint(y[3]);
    return v;
  }
  __device__ static __forceinline__ void store1(char* rowp, int64_t idx, float y) {
    reinterpret_cast<float*>(rowp)[idx] = y;
  }
};

template <>
struct ElemOut<1> {
  __device__ static __forceinline__ uint32_t pack2(float lo, float hi) {
    const f32x2 v = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2));  // round to nearest even
  }
  __device__ static __forceinline__ u32x4 pack(const float* y) {
    u32x4 v;
    v.x = pack2(y[0], y[1]);
    v.y = pack2(y[2], y[3]);
    v.z = pack2(y[4], y[5]);
    v.w = pack2(y[6], y[7]);
    return v;
  }
  __device__ static __forceinline__ void store1(char* rowp, int64_t idx, float y) {
    reinterpret_cast<uint16_t*>(rowp)[idx] = static_cast<uint16_t>(pack2(y, 0.f) & 0xffffu);
  }
};

template <>
struct ElemOut<2> {
  typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
  __device__ static __forceinline__ uint32_t pack2(float lo, float hi) {
    const f32x2 v = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, f16x2));  // round to nearest even
  }
  __device__ static __forceinline__ u32x4 pack(const float* y) {
    u32x4 v;
    v.x = pack2(y[0], y[1]);
    v.y = pack2(y[2], y[3]);
    v.z = pack2(y[4], y[5]);
    v.w = pack2(y[6], y[7]);
    return v;
  }
  __device__ static __forceinline__ void store1(char* rowp, int64_t idx, float y) {
    reinterpret_cast<_Float16*>(rowp)[idx] = static_cast<_Float16>(y);
  }
};

struct RowGrad {
  float c;     // log2e / T
  float lse2;  // lse * log2e
  float a;     // -g_h * ln2 / T
  float b;     // -(g_l + g_h * H) / T
  float lab;   // g_l / T, added at the label
  __device__ __forceinline__ float operator()(float x) const {
    const float u = __builtin_fmaf(x, c, -lse2);
    const float p = hw_exp2(u);
    // p == 0 (a -inf logit, or one far below the row's bulk) has zero gradient; without the
    // select, u = -inf would give 0 * inf.
    return (p == 0.f) ? 0.f : p * __builtin_fmaf(u, a, b);
  }
};

// The fp32 form: the quotient and log p are formed like torch forms them.
struct RowGradExact {
  Scale<true> sc;  // T, RN(1/T)
  float lse;
  float a;    // -g_h / T
  float b;    // -(g_l + g_h * H) / T
  float lab;  // g_l / T, added at the label
  __device__ __forceinline__ float operator()(float x) const {
    const float d = sc.pre(x) - lse;  // log p
    const float p = hw_exp2(d * kLog2e);
    return (p == 0.f) ? 0.f : p * __builtin_fmaf(d, a, b);
  }
};

// The whole workgroup (WAVES*64 threads) writes the gradient of one row: out[v] = f(in[v]) (+ f.lab at v == label).
// Rows need not be 16-byte aligned; the vector path is taken when input and output rows share their 16-byte phase.
template <int DT, int WAVES, int U, class F>
__device__ __forceinline__ void backward_row(const char* rowp, char* outp, int64_t vocab, const F& f, int64_t label) {
  using E = Elem<DT>;
  using O = ElemOut<DT>;
  constexpr int NTHR = WAVES * 64;
  constexpr int PV = E::kPerVec;
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const uintptr_t ain = reinterpret_cast<uintptr_t>(rowp);
  const uintptr_t aout = reinterpret_cast<uintptr_t>(outp);
  const bool same_phase = ((ain ^ aout) & 15u) == 0;
  int64_t head = same_phase ? static_cast<int64_t>(((16u - (ain & 15u)) & 15u) / E::kBytes) : vocab;
  if (head > vocab) head = vocab;
  const int64_t nvec = (vocab - head) / PV;
  const int64_t tail0 = head + nvec * PV;
  const u32x4* vin = reinterpret_cast<const u32x4*>(rowp + head * E::kBytes);
  u32x4* vout = reinterpret_cast<u32x4*>(outp + head * E::kBytes);

  auto do_vec = [&](int64_t k, const u32x4& v) {
    float x[PV];
    E::unpack(v, x);
#pragma unroll
    for (int i = 0; i < PV; ++i) x[i] = f(x[i]);
    const int64_t rel = label - (head + k * PV);
    if (rel >= 0 && rel < PV) {
#pragma unroll
      for (int i = 0; i < PV; ++i)
        if (i == rel) x[i] += f.lab;
    }
    __builtin_nontemporal_store(O::pack(x), vout + k);
  };

  constexpr int64_t kBatchVecs = static_cast<int64_t>(NTHR) * U;
  const int64_t nfull = nvec / kBatchVecs;
  for (int64_t j = 0; j < nfull; ++j) {
    const int64_t k0 = (j * WAVES + wave) * (U * 64) + lane;
    u32x4 v[U];
#pragma unroll
    for (int u = 0; u < U; ++u) v[u] = __builtin_nontemporal_load(vin + k0 + u * 64);
#pragma unroll
    for (int u = 0; u < U; ++u) do_vec(k0 + u * 64, v[u]);
  }
  for (int64_t k = nfull * kBatchVecs + tid; k < nvec; k += NTHR) do_vec(k, __builtin_nontemporal_load(vin + k));

  // scalars: [0, head) and [tail0, vocab); with mismatched phases that is the whole row
  for (int64_t i = tid; i < head + (vocab - tail0); i += NTHR) {
    const int64_t idx = (i < head) ? i : tail0 + (i - head);
    float y = f(E::load1(rowp, idx));
    if (idx == label) y += f.lab;
    O::store1(outp, idx, y);
  }
}

// The whole workgroup fills one output row with zeros without reading anything.
template <int DT, int WAVES>
__device__ __forceinline__ void zero_row(char* outp, int64_t vocab) {
  using E = Elem<DT>;
  using O = ElemOut<DT>;
  constexpr int NTHR = WAVES * 64;
  constexpr int PV = E::kPerVec;
  const int tid = threadIdx.x;
  const uintptr_t aout = reinterpret_cast<uintptr_t>(outp);
  int64_t head = static_cast<int64_t>(((16u - (aout & 15u)) & 15u) / E::kBytes);
  if (head > vocab) head = vocab;
  const int64_t nvec = (vocab - head) / PV;
  const int64_t tail0 = head + nvec * PV;
  u32x4* vout = reinterpret_cast<u32x4*>(outp + head * E::kBytes);
  const u32x4 z = {0u, 0u, 0u, 0u};
  for (int64_t k = tid; k < nvec; k += NTHR) __builtin_nontemporal_store(z, vout + k);
  for (int64_t i = tid; i < head + (vocab - tail0); i += NTHR) O::store1(outp, (i < head) ? i : tail0 + (i - head), 0.f);
}

// The row constants of the gradient from what the forward pass left and the incoming gradients.
template <bool EXACT>
__device__ __forceinline__ typename std::conditional<EXACT, RowGradExact, RowGrad>::type make_row_grad(
    float T, float lse, float H, float gl, float gh) {
  typename std::conditional<EXACT, RowGradExact, RowGrad>::type f;
  const float rT = 1.0f / T;
  if constexpr (EXACT) {
    f.sc.c = kLog2e;
    f.sc.T = T;
    f.sc.r = rT;
    f.lse = lse;
    f.a = -gh * rT;
  } else {
    f.c = kLog2e * rT;
    f.lse2 = lse * kLog2e;
    f.a = -(gh * kLn2f) * rT;
  }
  f.b = -(gl + gh * H) * rT;
  f.lab = gl * rT;
  return f;
}

// grid.x = n_rows, block = WAVES*64. EXACT selects RowGradExact (fp32 logits).
template <int DT, int WAVES, int U, bool EXACT = (DT == 0)>
__global__ __launch_bounds__(WAVES * 64) void rowscore_backward_kernel(
    const void* logits, int64_t vocab, int64_t row_stride, const int64_t* __restrict__ labels,
    const float* __restrict__ temperature, const float* __restrict__ lse, const float* __restrict__ entropy,
    const float* __restrict__ g_logprob, const float* __restrict__ g_entropy, void* dlogits,
    int64_t d_row_stride) {
  using E = Elem<DT>;
  const int64_t row = blockIdx.x;
  const char* rowp = static_cast<const char*>(logits) + row * row_stride * E::kBytes;
  char* outp = static_cast<char*>(dlogits) + row * d_row_stride * E::kBytes;

  float T = 1.f;
  if (temperature != nullptr) {
    T = temperature[row];
    T = (T < kMinTemperature) ? kMinTemperature : T;
  }
  const float gl = (g_logprob != nullptr) ? g_logprob[row] : 0.f;
  const float gh = (g_entropy != nullptr) ? g_entropy[row] : 0.f;
  const float H = (g_entropy != nullptr) ? entropy[row] : 0.f;
  const auto f = make_row_grad<EXACT>(T, lse[row], H, gl, gh);
  // a label outside [0, vocab) was reported by the forward pass; here it simply matches nothing
  const int64_t label = (g_logprob != nullptr) ? labels[row] : -1;
  backward_row<DT, WAVES, U>(rowp, outp, vocab, f, label);
}

// The same gradient for rows that lie back to back (row pitch = vocabulary, input and output) on 16-byte boundaries,
// without a workgroup per row: workgroups of 4 wavefronts walk the rows as one array, a wavefront moving 8 KiB per trip
// (8 non-temporal 128-bit loads per lane, then 8 stores), a workgroup as many trips as the host's grid leaves it. On
// this part a read + write stream in that form runs 7 % (bf16) to 20 % (fp32) faster than one workgroup per row. A trip
// (512 vectors) touches at most two rows, since a row holds at least 512 vectors: the row constants of both are formed
// per trip and a lane picks by its vector's position. The arithmetic per element is rowscore_backward_kernel's, so the
// results are the same bits.
constexpr int kFlatBackwardThreads = 256;
constexpr int kFlatBackwardUnroll = 8;
constexpr int64_t kFlatBackwardTripVecs = 64 * kFlatBackwardUnroll;   // per wavefront and trip

// The walk itself. row_constants(r, &label, &active) gives the gradient's constants of row r (wave-uniform r; called by
// the whole wavefront): `active` false means the row's gradient is zero and its logits are not to be read.
template <int DT, class RowConstants>
__device__ __forceinline__ void backward_flat_walk(const void* logits, int64_t n_rows, int64_t vocab, void* dlogits,
                                                   RowConstants&& row_constants) {
  using E = Elem<DT>;
  using O = ElemOut<DT>;
  constexpr int PV = E::kPerVec;
  constexpr int U = kFlatBackwardUnroll;
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(static_cast<int>(threadIdx.x >> 6));
  const int64_t row_vecs = vocab / PV;   // the host passes a multiple of PV, at least kFlatBackwardTripVecs vectors
  const int64_t nvec = n_rows * row_vecs;
  const u32x4* vin = static_cast<const u32x4*>(logits);
  u32x4* vout = static_cast<u32x4*>(dlogits);
  // a workgroup's trips lie a whole grid apart (measured against consecutive ones: 883 against 899-944 us at 8192 x 151936
  // bf16 with two to eight trips per workgroup)
  const int64_t stride = static_cast<int64_t>(gridDim.x) * (kFlatBackwardThreads / 64) * kFlatBackwardTripVecs;
  const int64_t stride_rows = stride / row_vecs, stride_rem = stride % row_vecs;
  int64_t base = (static_cast<int64_t>(blockIdx.x) * (kFlatBackwardThreads / 64) + wave) * kFlatBackwardTripVecs;
  int64_t row = base / row_vecs, rem = base % row_vecs;   // the trip's first vector: vector `rem` of row `row`

  for (; base < nvec; base += stride) {
    int64_t label0, label1;
    bool active0, active1;
    const auto f0 = row_constants(row, &label0, &active0);
    const auto f1 = row_constants(row + 1 < n_rows ? row + 1 : row, &label1, &active1);
    u32x4 v[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int64_t k = base + u * 64 + lane;
      const bool active = (rem + u * 64 + lane >= row_vecs) ? active1 : active0;
      v[u] = (k < nvec && active) ? __builtin_nontemporal_load(vin + k) : u32x4{0u, 0u, 0u, 0u};
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int64_t k = base + u * 64 + lane;
      const int64_t in_row = rem + u * 64 + lane;       // vector index counted from the first row's start
      const bool second = in_row >= row_vecs;
      const auto f = second ? f1 : f0;
      const int64_t first_elem = (second ? in_row - row_vecs : in_row) * PV;
      const int64_t rel = (second ? label1 : label0) - first_elem;
      float x[PV];
      E::unpack(v[u], x);
#pragma unroll
      for (int i = 0; i < PV; ++i) x[i] = f(x[i]);
      if (rel >= 0 && rel < PV) {
#pragma unroll
        for (int i = 0; i < PV; ++i)
          if (i == rel) x[i] += f.lab;
      }
      u32x4 y = O::pack(x);
      if (!(second ? active1 : active0)) y = u32x4{0u, 0u, 0u, 0u};
      if (k < nvec) __builtin_nontemporal_store(y, vout + k);
    }
    row += stride_rows;
    rem += stride_rem;
    if (rem >= row_vecs) {
      rem -= row_vecs;
      ++row;
    }
  }
}

template <int DT, bool EXACT = (DT == 0)>
__global__ __launch_bounds__(kFlatBackwardThreads) void rowscore_backward_flat_kernel(
    const void* logits, int64_t n_rows, int64_t vocab, const int64_t* __restrict__ labels,
    const float* __restrict__ temperature, const float* __restrict__ lse, const float* __restrict__ entropy,
    const float* __restrict__ g_logprob, const float* __restrict__ g_entropy, void* dlogits) {
  backward_flat_walk<DT>(logits, n_rows, vocab, dlogits, [&](int64_t r, int64_t* label, bool* active) {
    float T = 1.f;
    if (temperature != nullptr) {
      T = temperature[r];
      T = (T < kMinTemperature) ? kMinTemperature : T;
    }
    const float gl = (g_logprob != nullptr) ? g_logprob[r] : 0.f;
    const float gh = (g_entropy != nullptr) ? g_entropy[r] : 0.f;
    const float H = (g_entropy != nullptr) ? entropy[r] : 0.f;
    *label = (g_logprob != nullptr) ? labels[r] : -1;   // one outside [0, vocab) matches nothing
    *active = true;
    return make_row_grad<EXACT>(T, lse[r], H, gl, gh);
  });
}

// The gradient of score_responses_kernel in the same form, for batches of at most 64 sequences (a wavefront finds a
// row's sequence with one pair of loads per lane and a ballot instead of a bisection per trip): rows outside every
// response window, and rows of sequences that fail validation, are written as zeros without being read, like
// score_responses_backward_kernel below, and the rows inside get the same bits as there.
template <int DT, bool EXACT = (DT == 0)>
__global__ __launch_bounds__(kFlatBackwardThreads) void score_responses_backward_flat_kernel(
    const void* logits, int64_t n_rows, int64_t vocab, const int64_t* __restrict__ labels,
    const int64_t* __restrict__ input_ids, const float* __restrict__ temperature,
    const int64_t* __restrict__ cu_seqlens, const int64_t* __restrict__ response_lens, int64_t B, int64_t T_out,
    const float* __restrict__ resp_lse, const float* __restrict__ resp_entropy,
    const float* __restrict__ g_resp_logprob, const float* __restrict__ g_resp_entropy, void* dlogits) {
  const int lane = threadIdx.x & 63;
  backward_flat_walk<DT>(logits, n_rows, vocab, dlogits, [&](int64_t r, int64_t* label, bool* active) {
    *label = -1;
    *active = false;
    bool hit = false;
    if (lane < B) hit = cu_seqlens[lane] <= r && r < cu_seqlens[lane + 1];
    const unsigned long long holders = __ballot(hit);
    int64_t at = 0;
    if (holders != 0ull) {
      const int64_t b = __builtin_ctzll(holders);
      int why = 0;
      const ResponseWindow w = response_window(cu_seqlens, response_lens, b, B, n_rows, T_out, &why);
      const int64_t col = r - w.first;
      if (w.ok && col >= 0 && col < w.resp) {
        *active = true;
        at = b * T_out + col;
      }
    }
    float T = 1.f, gl = 0.f, gh = 0.f, H = 0.f, l = 0.f;
    if (*active) {
      if (temperature != nullptr) {
        T = temperature[r];
        T = (T < kMinTemperature) ? kMinTemperature : T;
      }
      gl = (g_resp_logprob != nullptr) ? g_resp_logprob[at] : 0.f;
      gh = (g_resp_entropy != nullptr) ? g_resp_entropy[at] : 0.f;
      H = (g_resp_entropy != nullptr) ? resp_entropy[at] : 0.f;
      l = resp_lse[at];
      if (g_resp_logprob != nullptr)
        *label = (input_ids != nullptr) ? input_ids[r + 1 < n_rows ? r + 1 : 0] : labels[r];
    }
    return make_row_grad<EXACT>(T, l, H, gl, gh);
  });
}

// Backward of score_responses_kernel (rowscore_kernels.h). grid.x = n_rows, block = WAVES*64. Row r finds its
// sequence by bisection like the forward kernel; inside a valid response window it reads the forward's logsumexp and
// entropy and the incoming gradients at (b, col) of the (B, T_out) blocks and writes its gradient row; every other row
// (prompts, sequences that failed validation, rows no sequence owns) gets zeros without its logits being read.
template <int DT, int WAVES, int U, bool EXACT = (DT == 0)>
__global__ __launch_bounds__(WAVES * 64) void score_responses_backward_kernel(
    const void* logits, int64_t n_rows, int64_t vocab, int64_t row_stride, const int64_t* __restrict__ labels,
    const int64_t* __restrict__ input_ids, const float* __restrict__ temperature,
    const int64_t* __restrict__ cu_seqlens, const int64_t* __restrict__ response_lens, int64_t B, int64_t T_out,
    const float* __restrict__ resp_lse, const float* __restrict__ resp_entropy,
    const float* __restrict__ g_resp_logprob, const float* __restrict__ g_resp_entropy, void* dlogits,
    int64_t d_row_stride) {
  using E = Elem<DT>;
  const int64_t row = blockIdx.x;
  char* outp = static_cast<char*>(dlogits) + row * d_row_stride * E::kBytes;
  int64_t lo = 0, hi = B;
  while (hi - lo > 1) {
    const int64_t mid = (lo + hi) >> 1;
    if (cu_seqlens[mid] <= row) lo = mid; else hi = mid;
  }
  const int64_t b = lo;
  bool in_window = false;
  int64_t col = 0;
  if (B > 0 && cu_seqlens[b] <= row && row < cu_seqlens[b + 1]) {
    int why = 0;
    const ResponseWindow w = response_window(cu_seqlens, response_lens, b, B, n_rows, T_out, &why);
    if (w.ok) {
      col = row - w.first;
      in_window = col >= 0 && col < w.resp;
    }
  }
  if (!in_window) {   // the whole workgroup
    zero_row<DT, WAVES>(outp, vocab);
    return;
  }
  const char* rowp = static_cast<const char*>(logits) + row * row_stride * E::kBytes;
  float T = 1.f;
  if (temperature != nullptr) {
    T = temperature[row];
    T = (T < kMinTemperature) ? kMinTemperature : T;
  }
  const int64_t at = b * T_out + col;
  const float gl = (g_resp_logprob != nullptr) ? g_resp_logprob[at] : 0.f;
  const float gh = (g_resp_entropy != nullptr) ? g_resp_entropy[at] : 0.f;
  const float H = (g_resp_entropy != nullptr) ? resp_entropy[at] : 0.f;
  const auto f = make_row_grad<EXACT>(T, resp_lse[at], H, gl, gh);
  int64_t label = -1;
  if (g_resp_logprob != nullptr) label = (input_ids != nullptr) ? input_ids[row + 1 < n_rows ? row + 1 : 0] : labels[row];
  backward_row<DT, WAVES, U>(rowp, outp, vocab, f, label);
}

}  // namespace vrl
