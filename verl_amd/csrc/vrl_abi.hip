// C ABI of libvrl_hip.so: argument checks on the host, then kernel launches on
// the caller's stream. Declarations and the reference interfaces each entry
// point replaces are in include/vrl.h.
#include "vrl.h"

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <string.h>

#include <atomic>

#include "backward_kernels.h"
#include "layout_kernels.h"
#include "lmhead_kernels.h"
#include "rollout_corr_kernels.h"
#include "row_shapes.h"
#include "rowscore_kernels.h"
#include "transpose_kernels.h"
#include "verify_flat_kernels.h"
#include "verify_kernels.h"

namespace {

thread_local char g_hip_error[256] = {0};

int launch_status() {
  const hipError_t e = hipGetLastError();
  if (e == hipSuccess) return VRL_OK;
  const char* msg = hipGetErrorString(e);
  strncpy(g_hip_error, msg ? msg : "unknown HIP error", sizeof(g_hip_error) - 1);
  g_hip_error[sizeof(g_hip_error) - 1] = 0;
  return VRL_ERR_HIP;
}

bool aligned(const void* p, uintptr_t a) { return (reinterpret_cast<uintptr_t>(p) & (a - 1)) == 0; }

bool known_dtype(int dtype) { return dtype == VRL_F32 || dtype == VRL_BF16 || dtype == VRL_F16; }

constexpr int64_t kMaxGrid = 0x7fffffffLL;

// Device-resident scratch of vrl_rowscore_split_static: VRL_STATIC_PARTIALS_MAX (row, slice) partials of 4 floats.
// Each GPU the library runs on holds its own copy of this array at its own address until the process ends. On the
// host the name `scratch` is only a handle for hipGetSymbolAddress, never a device address: kernels and copies get
// the per-device pointer that static_scratch() looks up once per device.
static __device__ __align__(256) float scratch[VRL_STATIC_PARTIALS_MAX * 4];

constexpr int kMaxDevices = 64;
std::atomic<float*> g_scratch_ptr[kMaxDevices];

int check_rowscore(const void* logits, int dtype, int64_t n_rows, int64_t vocab, int64_t row_stride,
                   const int64_t* labels, const float* temperature, const float* out_logprob,
                   const float* out_entropy, const float* out_sum_pi_sq, const float* out_lse,
                   const int32_t* err_flag) {
  if (!known_dtype(dtype)) return VRL_ERR_DTYPE;
  if (n_rows < 0 || vocab <= 0 || row_stride < vocab || n_rows > kMaxGrid) return VRL_ERR_SHAPE;
  if (out_logprob == nullptr && out_entropy == nullptr && out_sum_pi_sq == nullptr && out_lse == nullptr)
    return VRL_ERR_ARG;
  if (n_rows == 0) return VRL_OK;
  if (logits == nullptr) return VRL_ERR_NULL;
  if (out_logprob != nullptr && (labels == nullptr || err_flag == nullptr)) return VRL_ERR_NULL;
  const uintptr_t esize = (dtype == VRL_F32) ? 4 : 2;
  if (!aligned(logits, esize) || !aligned(labels, 8) || !aligned(temperature, 4) ||
      !aligned(out_logprob, 4) || !aligned(out_entropy, 4) || !aligned(out_sum_pi_sq, 4) ||
      !aligned(out_lse, 4) || !aligned(err_flag, 4))
    return VRL_ERR_ALIGN;
  return VRL_OK;
}

struct RowArgs {
  const void* logits;
  int64_t n_rows, vocab, row_stride;
  const int64_t* labels;
  const float* temperature;
  float* out_logprob;
  float* out_entropy;
  float* out_sum_pi_sq;
  float* out_lse;
  int32_t* err_flag;
  int n_splits;     // 1: one workgroup per row
  float* partials;  // split path only
  hipStream_t stream;
};

int64_t split_slice_elems(int64_t vocab, int n_splits, int dtype) {
  const int64_t per_vec = (dtype == VRL_F32) ? 4 : 8;
  const int64_t batch = static_cast<int64_t>(kSplitWaves) * 64 * kSplitUnroll * per_vec;
  const int64_t per_split = (vocab + n_splits - 1) / n_splits;
  return ((per_split + batch - 1) / batch) * batch;
}

// Launches of fewer rows than this end in a long tail when many workgroups share a CU (the last rows
// each get a fraction of the CU's bandwidth); 16-wavefront workgroups keep two rows per CU in flight
// and halve that tail. Measured at 8192 x 151936 bf16: 7.01 TB/s against 6.80; at 32768 rows the
// 8-wavefront shape is ahead (6.99 against 6.85).
constexpr int64_t kWideRowsBelow = 16384;
constexpr int64_t kWideVocabFrom = 16384;  // shorter rows would leave most of 1024 lanes without a vector

// Address of `scratch` on the current device (looked up on the first call per device; two threads racing through the
// first call store the same value).
int static_scratch(float** out) {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess) return launch_status();
  if (dev < 0 || dev >= kMaxDevices) return VRL_ERR_SHAPE;
  float* p = g_scratch_ptr[dev].load(std::memory_order_acquire);
  if (p == nullptr) {
    void* sym = nullptr;
    if (hipGetSymbolAddress(&sym, HIP_SYMBOL(scratch)) != hipSuccess || sym == nullptr) {
      const int st = launch_status();
      return st != VRL_OK ? st : VRL_ERR_HIP;
    }
    p = static_cast<float*>(sym);
    g_scratch_ptr[dev].store(p, std::memory_order_release);
  }
  *out = p;
  return VRL_OK;
}

template <int DT, int W, int U, bool EXACT, bool WANT_Q>
void launch_row_kernel(const RowArgs& a) {
  vrl::rowscore_kernel<DT, W, U, EXACT, true, WANT_Q>
      <<<dim3(static_cast<unsigned>(a.n_rows)), dim3(W * 64), 0, a.stream>>>(
          a.logits, a.vocab, a.row_stride, a.labels, a.temperature, a.out_logprob, a.out_entropy,
          a.out_sum_pi_sq, a.out_lse, a.err_flag);
}

template <int DT, bool EXACT, bool WANT_Q>
void launch_rows(const RowArgs& a) {
  if (a.n_splits <= 1) {
    if (a.n_rows < kWideRowsBelow && a.vocab >= kWideVocabFrom)
      launch_row_kernel<DT, 16, 2, EXACT, WANT_Q>(a);
    else
      launch_row_kernel<DT, RowShape<DT>::kWaves, RowShape<DT>::kUnroll, EXACT, WANT_Q>(a);
    return;
  }
  const int64_t slice = split_slice_elems(a.vocab, a.n_splits, DT);
  vrl::rowscore_split_kernel<DT, kSplitWaves, kSplitUnroll, EXACT, true, WANT_Q>
      <<<dim3(static_cast<unsigned>(a.n_rows * a.n_splits)), dim3(kSplitWaves * 64), 0, a.stream>>>(
          a.logits, a.vocab, a.row_stride, a.temperature, a.n_splits, slice, a.partials);
  vrl::rowscore_merge_kernel<DT, EXACT, WANT_Q>
      <<<dim3(static_cast<unsigned>((a.n_rows + 63) / 64)), dim3(64), 0, a.stream>>>(
          a.logits, a.n_rows, a.vocab, a.row_stride, a.labels, a.temperature, a.n_splits, a.partials,
          a.out_logprob, a.out_entropy, a.out_sum_pi_sq, a.out_lse, a.err_flag);
}

template <int DT, bool EXACT>
void launch_rows_q(const RowArgs& a) {
  if (a.out_sum_pi_sq != nullptr)
    launch_rows<DT, EXACT, true>(a);
  else
    launch_rows<DT, EXACT, false>(a);
}

void launch_rows_any(int dtype, const RowArgs& a) {
  if (dtype == VRL_F32) {
    // fp32 logits with a temperature: per-element quotient rounded like `logits / temperature`
    if (a.temperature != nullptr)
      launch_rows_q<VRL_F32, true>(a);
    else
      launch_rows_q<VRL_F32, false>(a);
  } else if (dtype == VRL_BF16) {
    launch_rows_q<VRL_BF16, false>(a);
  } else {
    launch_rows_q<VRL_F16, false>(a);
  }
}

// Size rules of the sequence space: padded (B, T) arrays hold exactly B*T tokens; packed arrays hold n_tokens and
// the device-side offsets are checked against it by the kernels, which need somewhere to report to.
int check_layout(const int64_t* cu_seqlens, int64_t B, int64_t T, int64_t n_tokens, const int32_t* err_flag) {
  if (B < 0 || T < 0 || n_tokens < 0 || B > kMaxGrid || T > kMaxGrid) return VRL_ERR_SHAPE;
  if (cu_seqlens == nullptr) {
    if (n_tokens != B * T) return VRL_ERR_SHAPE;
  } else if (B > 0 && err_flag == nullptr) {
    return VRL_ERR_NULL;
  }
  if (!aligned(cu_seqlens, 8) || !aligned(err_flag, 4)) return VRL_ERR_ALIGN;
  return VRL_OK;
}

template <int DT, int W, int U, bool EXACT>
void launch_score_responses(const void* logits, int64_t n_rows, int64_t vocab, int64_t row_stride,
                            const int64_t* labels, const int64_t* input_ids, const float* temperature,
                            const int64_t* cu_seqlens, const int64_t* response_lens, int64_t B, int64_t T_out,
                            float* out_logprob, float* out_entropy, float* resp_logprob, float* resp_entropy,
                            float* resp_lse, int32_t* err_flag, hipStream_t s) {
  vrl::score_responses_kernel<DT, W, U, EXACT><<<dim3(static_cast<unsigned>(n_rows + B)), dim3(W * 64), 0, s>>>(
      logits, n_rows, vocab, row_stride, labels, input_ids, temperature, cu_seqlens, response_lens, B, T_out,
      out_logprob, out_entropy, resp_logprob, resp_entropy, resp_lse, err_flag);
}

template <int DT, bool EXACT, typename... Args>
void launch_score_responses_shaped(int64_t n_rows, int64_t vocab, Args... a) {
  // same workgroup shapes as the plain row kernel (see launch_rows)
  if (n_rows < kWideRowsBelow && vocab >= kWideVocabFrom)
    launch_score_responses<DT, 16, 2, EXACT>(a...);
  else
    launch_score_responses<DT, RowShape<DT>::kWaves, RowShape<DT>::kUnroll, EXACT>(a...);
}

int check_verify(const float* logp_new, const float* logp_old, const float* log_u, const uint8_t* mask,
                 const int64_t* cu_seqlens, int64_t B, int64_t T, int64_t n_tokens, const int32_t* err_flag,
                 const uint8_t* accept, const int32_t* first_reject, const int32_t* prefix_len,
                 const int32_t* near_count, const int64_t* draft_ids, const int64_t* out_ids,
                 const uint8_t* out_mask) {
  (void)mask;
  const int ls = check_layout(cu_seqlens, B, T, n_tokens, err_flag);
  if (ls != VRL_OK) return ls;
  const bool any_trunc = (draft_ids != nullptr) || (out_ids != nullptr) || (out_mask != nullptr);
  const bool all_trunc = (draft_ids != nullptr) && (out_ids != nullptr) && (out_mask != nullptr);
  if (any_trunc && !all_trunc) return VRL_ERR_ARG;
  if (B == 0) return VRL_OK;
  if (first_reject == nullptr || prefix_len == nullptr || near_count == nullptr) return VRL_ERR_NULL;
  // Without tokens the kernel only writes the per-sequence zeros.
  const bool has_tokens = n_tokens > 0;
  if (has_tokens && (logp_new == nullptr || logp_old == nullptr || log_u == nullptr || accept == nullptr))
    return VRL_ERR_NULL;
  if (!aligned(logp_new, 4) || !aligned(logp_old, 4) || !aligned(log_u, 4) || !aligned(cu_seqlens, 8) ||
      !aligned(first_reject, 4) || !aligned(prefix_len, 4) || !aligned(near_count, 4) ||
      !aligned(draft_ids, 8) || !aligned(out_ids, 8))
    return VRL_ERR_ALIGN;
  return VRL_OK;
}

// From this many tokens on vrl_spec_verify_plan recommends the two flat passes (packed layout; padded: with at least
// kFlatMinPaddedT tokens per sequence and fewer than two sequences per CU as well).
constexpr int64_t kFlatMinTokens = 131072;
constexpr int64_t kFlatMinPaddedT = 4096;

// Wavefronts per sequence for the verify/truncate kernels. A workgroup handles 4 * 64 * waves tokens per
// memory round trip; long sequences want many wavefronts, a batch of many short ones wants few (idle
// wavefronts still have to be launched). Packed layouts keep their lengths on the device, so the
// choice there goes by the number of sequences.
int verify_waves(const int64_t* cu_seqlens, int64_t B, int64_t T) {
  if (cu_seqlens == nullptr) return T <= 256 ? 1 : (T <= 2048 ? 4 : 16);
  return B <= 4096 ? 16 : 4;
}

// Response slicing moves rows of `row_bytes` bytes in units of the largest power of two up to 16 that divides the row
// and the alignment of both arrays.
constexpr int64_t kMaxRowBytes = int64_t(1) << 30;
constexpr int64_t kMaxGridY = 65535;
constexpr int64_t kPackMaxChunks = 64;

int copy_unit(int64_t row_bytes, const void* a, const void* b) {
  for (int u = 16; u > 1; u >>= 1)
    if (row_bytes % u == 0 && aligned(a, u) && aligned(b, u)) return u;
  return 1;
}

struct LmGrid {
  int64_t tblocks;
  int tiles_per_split;
  int64_t grid;    // workgroups, the idle ones at its end included
};

// `run` tiles at a time go to a split: kLmSubTiles for the forward kernel, which hands its softmax state over at the
// ends of such runs, 1 for the gradient kernel, whose results are elementwise.
LmGrid lm_grid(int64_t T, int64_t V, int n_splits, int run) {
  LmGrid g;
  g.tblocks = (T + vrl::kLmTokens - 1) / vrl::kLmTokens;
  const int64_t vtiles = (V + vrl::kLmVocab - 1) / vrl::kLmVocab;
  const int64_t runs = (vtiles + run - 1) / run;
  g.tiles_per_split = static_cast<int>((runs + n_splits - 1) / n_splits) * run;
  g.grid = vrl::lm_dealt_grid(g.tblocks * n_splits);
  return g;
}

// The matrix-core kernels ask for more LDS than the default limit: raise it once per device and kernel, not per launch.
int raise_lds_limit(const void* kernel, std::atomic<bool>* raised) {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess) return launch_status();
  if (dev < 0 || dev >= kMaxDevices) return VRL_ERR_SHAPE;
  if (!raised[dev].load(std::memory_order_acquire)) {
    if (hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, vrl::kLmLdsBytes) != hipSuccess)
      return launch_status();
    raised[dev].store(true, std::memory_order_release);
  }
  return VRL_OK;
}

template <int DT, bool STORE>
int launch_lmhead(const void* hidden, const void* weight, int64_t T, int64_t V, int64_t K, int64_t h_stride,
                  int64_t w_stride, const int64_t* labels, const float* temperature, int n_splits, float* partials,
                  float* out_logprob, float* out_entropy, float* out_lse, int32_t* err_flag, void* logits_out,
                  int64_t l_stride, int64_t l_rows, hipStream_t s) {
  const LmGrid g = lm_grid(T, V, n_splits, vrl::kLmSubTiles);
  static std::atomic<bool> raised[kMaxDevices];
  const int rs = raise_lds_limit(reinterpret_cast<const void*>(vrl::lmhead_partial_kernel<DT, STORE>), raised);
  if (rs != VRL_OK) return rs;
  vrl::lmhead_partial_kernel<DT, STORE><<<dim3(static_cast<unsigned>(g.grid)), dim3(vrl::kLmWaves * 64),
                                          vrl::kLmLdsBytes, s>>>(
      static_cast<const uint16_t*>(weight), static_cast<const uint16_t*>(hidden), V, T, K, w_stride, h_stride,
      temperature, n_splits, g.tiles_per_split, partials, static_cast<uint16_t*>(logits_out), l_stride,
      l_rows);
  vrl::lmhead_finish_kernel<DT><<<dim3(static_cast<unsigned>((T + 3) / 4)), dim3(256), 0, s>>>(
      static_cast<const char*>(weight), static_cast<const char*>(hidden), V, T, K, w_stride, h_stride, labels,
      temperature, static_cast<int>((((V + vrl::kLmVocab - 1) / vrl::kLmVocab) + vrl::kLmSubTiles - 1) / vrl::kLmSubTiles),
      partials, out_logprob, out_entropy, out_lse, err_flag);
  return launch_status();
}

template <int DT>
int launch_lmhead_dlogits(const void* hidden, const void* weight, int64_t T, int64_t V, int64_t K, int64_t h_stride,
                          int64_t w_stride, const int64_t* labels, const float* temperature, const float* lse,
                          const float* entropy, const float* g_logprob, const float* g_entropy, int n_splits,
                          void* dlogits, int64_t d_stride, hipStream_t s) {
  const LmGrid g = lm_grid(T, V, n_splits, 1);
  static std::atomic<bool> raised[kMaxDevices];
  const int rs = raise_lds_limit(reinterpret_cast<const void*>(vrl::lmhead_dlogits_kernel<DT>), raised);
  if (rs != VRL_OK) return rs;
  vrl::lmhead_dlogits_kernel<DT><<<dim3(static_cast<unsigned>(g.grid)), dim3(vrl::kLmWaves * 64),
                                   vrl::kLmLdsBytes, s>>>(
      static_cast<const uint16_t*>(weight), static_cast<const uint16_t*>(hidden), V, T, K, w_stride, h_stride, labels,
      temperature, lse, entropy, g_logprob, g_entropy, n_splits, g.tiles_per_split,
      static_cast<uint16_t*>(dlogits), d_stride);
  return launch_status();
}

// Shape rules the matrix-core kernels share.
// The matrix-core walk adds a lane's share of a load address (up to 7 rows + 128 bytes) as a 32-bit offset, and keeps
// row and column indices in 32-bit registers.
constexpr int64_t kLmMaxStride = int64_t(1) << 28;
constexpr int64_t kLmMaxRows = int64_t(1) << 30;

int check_lmhead_shape(int dtype, int64_t n_tokens, int64_t vocab, int64_t hidden_size, int64_t h_stride,
                       int64_t w_stride, int n_splits) {
  if (dtype != VRL_BF16 && dtype != VRL_F16) return VRL_ERR_DTYPE;
  if (h_stride > kLmMaxStride || w_stride > kLmMaxStride || vocab > kLmMaxRows || n_tokens > kLmMaxRows)
    return VRL_ERR_SHAPE;
  if (n_tokens < vrl::kLmTokens || vocab < vrl::kLmVocab || hidden_size <= 0 || hidden_size % vrl::kLmK != 0 ||
      h_stride < hidden_size || w_stride < hidden_size || h_stride % 8 != 0 || w_stride % 8 != 0 ||
      n_splits < 1 || n_splits > vrl::kLmMaxSplits)
    return VRL_ERR_SHAPE;
  if (vrl::lm_dealt_grid(((n_tokens + vrl::kLmTokens - 1) / vrl::kLmTokens) * n_splits) > kMaxGrid ||
      (n_tokens + 3) / 4 > kMaxGrid)
    return VRL_ERR_SHAPE;
  return VRL_OK;
}


// How vrl_gemm cuts its work: enough (y block, x split, contraction range) items to fill the part's CUs in whole
// rounds. One workgroup per CU runs at a time (the kernels take all of its LDS).
struct GemmPlan {
  vrl::LmGemmShape shape;
  int64_t patches;   // py x px groups of work items, over all contraction ranges
};

int device_cus() {
  static std::atomic<int> cus[kMaxDevices];
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return 256;
  int n = cus[dev].load(std::memory_order_acquire);
  if (n == 0) {
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
    cus[dev].store(n, std::memory_order_release);
  }
  return n;
}

// The workgroups resident on one XCD form patches of py y blocks x px x splits that walk the contraction in step and
// share operand tiles through its L2: an X tile is fetched once for the py workgroups that use it, a Y tile once for px,
// so what leaves L2 is proportional to 1/py + 1/px. Counts that py or px do not divide leave smaller patches in the
// last row or column, which lowers the sharing there; the choice below weighs both by the average number of
// workgroups per patch row and column. py <= 4, px <= 8: 32 CUs per XCD.
void choose_patch(int64_t nyb, int64_t nxs, int* py_out, int* px_out) {
  double best = 1e30;
  int best_py = 1, best_px = 1;
  for (int py = 1; py <= 4; ++py) {
    for (int px = 1; px <= 8; ++px) {
      const double eff_y = static_cast<double>(nyb) / static_cast<double>((nyb + py - 1) / py);
      const double eff_x = static_cast<double>(nxs) / static_cast<double>((nxs + px - 1) / px);
      const double slots = static_cast<double>(((nyb + py - 1) / py) * py) * static_cast<double>(((nxs + px - 1) / px) * px);
      // fetched bytes, and as a tie-break (1e-3 per unit) the share of slots that hold no work
      const double cost = 1.0 / eff_y + 1.0 / eff_x + 1e-3 * slots / (static_cast<double>(nyb) * static_cast<double>(nxs));
      if (cost < best - 1e-12) {
        best = cost;
        best_py = py;
        best_px = px;
      }
    }
  }
  *py_out = best_py;
  *px_out = best_px;
}

GemmPlan gemm_plan(int64_t NX, int64_t NY, int64_t K, int forced_parts) {
  GemmPlan p;
  vrl::LmGemmShape& g = p.shape;
  g.NX = NX;
  g.NY = NY;
  g.k_steps = K / vrl::kLmK;
  const int64_t nyb = (NY + vrl::kLmTokens - 1) / vrl::kLmTokens;
  const int64_t nxt = (NX + vrl::kLmVocab - 1) / vrl::kLmVocab;
  const int cus = device_cus();
  // x tiles per workgroup: 2 when that still leaves 8 rounds of work and a tile is at most 64 contraction steps (halves
  // the share of pipeline fill and drain; from 128 steps on the coarser items cost more in the last, partly filled round
  // than they save: d W at 8192 tokens 6.46 against 6.59 ms with one tile per item, the same at 4096)
  g.tiles_per_item = (nxt % 2 == 0 && nyb * (nxt / 2) >= 8LL * cus && g.k_steps <= 64) ? 2 : 1;
  const int64_t nxs = (nxt + g.tiles_per_item - 1) / g.tiles_per_item;
  const int64_t base = nyb * nxs;
  int best = 1;
  if (forced_parts > 0) {
    best = forced_parts;
  } else {
    // One workgroup per CU runs at a time, so a product takes (rounds of workgroups) x (contraction steps of a range, plus
    // a few to fill and drain the ring); cutting the contraction into ranges fills a last, nearly empty round at the
    // price of a pass over fp32 partial sums (a fixed cost and 8 bytes per output element and range, in units of a
    // 1.45 us step). Fitted to d hidden at 3584 <- 152064, one process: 8192 tokens 6.33 ms in 4 ranges against 6.63 in
    // one, 14080 tokens 11.6 in 6 against 13.4, 16384 tokens 12.9 in 2 against 14.6; 4096 tokens level (3.26 - 3.29).
    double best_cost = 0.0;
    for (int parts : {1, 2, 3, 4, 6, 8}) {
      if (parts > 1 && g.k_steps / parts < 32) break;
      const double rounds = static_cast<double>((base * parts + cus - 1) / cus);
      double cost = rounds * static_cast<double>((g.k_steps + parts - 1) / parts + 4);
      if (parts > 1) cost += 60.0 + 1.2e-6 * static_cast<double>(parts) * static_cast<double>(NX) * static_cast<double>(NY);
      if (parts == 1 || cost < 0.95 * best_cost) {   // more ranges only for a gain that is worth their scratch
        best_cost = cost;
        best = parts;
      }
    }
  }
  g.steps_per_part = static_cast<int>((g.k_steps + best - 1) / best);
  g.k_parts = static_cast<int>((g.k_steps + g.steps_per_part - 1) / g.steps_per_part);   // no empty range
  choose_patch(nyb, nxs, &g.py, &g.px);
  p.patches = ((nyb + g.py - 1) / g.py) * ((nxs + g.px - 1) / g.px) * g.k_parts;
  return p;
}

template <int DT, bool X_CM, bool Y_CM>
int launch_gemm(const void* x, const void* y, const GemmPlan& plan, int64_t x_stride, int64_t y_stride, void* out,
                int64_t out_stride, int accumulate, float* workspace, hipStream_t s) {
  const vrl::LmGemmShape& g = plan.shape;
  const int64_t grid = (plan.patches * g.py * g.px + 7) / 8 * 8;   // a slot per item of a full patch
  if (grid > kMaxGrid) return VRL_ERR_SHAPE;
  const dim3 gd(static_cast<unsigned>(grid)), bd(vrl::kLmWaves * 64);
  const uint16_t* X = static_cast<const uint16_t*>(x);
  const uint16_t* Y = static_cast<const uint16_t*>(y);
  uint16_t* O = static_cast<uint16_t*>(out);
#define VRL_GEMM_LAUNCH(MODE)                                                                                       \
  {                                                                                                                 \
    static std::atomic<bool> raised[kMaxDevices];                                                                   \
    const int rs =                                                                                                  \
        raise_lds_limit(reinterpret_cast<const void*>(vrl::lm_gemm_kernel<DT, MODE, X_CM, Y_CM>), raised);          \
    if (rs != VRL_OK) return rs;                                                                                    \
    vrl::lm_gemm_kernel<DT, MODE, X_CM, Y_CM><<<gd, bd, vrl::kLmLdsBytes, s>>>(X, Y, g, x_stride, y_stride, O,      \
                                                                               out_stride, workspace);              \
  }
  if (g.k_parts > 1) {
    VRL_GEMM_LAUNCH(2)
    const int64_t quads = g.NY * (g.NX / 4);
    const dim3 rg(static_cast<unsigned>((quads + 255) / 256));
    if (accumulate)
      vrl::lm_gemm_reduce_kernel<DT, true><<<rg, dim3(256), 0, s>>>(workspace, g.NX, g.NY, g.k_parts, O, out_stride);
    else
      vrl::lm_gemm_reduce_kernel<DT, false><<<rg, dim3(256), 0, s>>>(workspace, g.NX, g.NY, g.k_parts, O, out_stride);
  } else if (accumulate) {
    VRL_GEMM_LAUNCH(1)
  } else {
    VRL_GEMM_LAUNCH(0)
  }
#undef VRL_GEMM_LAUNCH
  return launch_status();
}

template <int DT>
int launch_gemm_layout(int x_cm, int y_cm, const void* x, const void* y, const GemmPlan& plan, int64_t x_stride,
                       int64_t y_stride, void* out, int64_t out_stride, int accumulate, float* workspace,
                       hipStream_t s) {
  if (x_cm && y_cm)
    return launch_gemm<DT, true, true>(x, y, plan, x_stride, y_stride, out, out_stride, accumulate, workspace, s);
  if (x_cm)
    return launch_gemm<DT, true, false>(x, y, plan, x_stride, y_stride, out, out_stride, accumulate, workspace, s);
  if (y_cm)
    return launch_gemm<DT, false, true>(x, y, plan, x_stride, y_stride, out, out_stride, accumulate, workspace, s);
  return launch_gemm<DT, false, false>(x, y, plan, x_stride, y_stride, out, out_stride, accumulate, workspace, s);
}

// A row-major operand is (N, K) with stride >= K; a contraction-major one is (K, N) with stride >= N and whole 16-byte
// groups of rows (N a multiple of 8).
int check_gemm(int dtype, int64_t NX, int64_t NY, int64_t K, int64_t x_stride, int64_t y_stride, int x_cm, int y_cm,
               int64_t out_stride) {
  if (dtype != VRL_BF16 && dtype != VRL_F16) return VRL_ERR_DTYPE;
  if (x_stride > kLmMaxStride || y_stride > kLmMaxStride || NX > kLmMaxRows || NY > kLmMaxRows || K > kLmMaxRows)
    return VRL_ERR_SHAPE;
  if (NX < vrl::kLmVocab || NY < vrl::kLmTokens || NX % 4 != 0 || K < 2 * vrl::kLmK || K % vrl::kLmK != 0 ||
      x_stride < (x_cm ? NX : K) || y_stride < (y_cm ? NY : K) || x_stride % 8 != 0 || y_stride % 8 != 0 ||
      (x_cm && NX % 8 != 0) || (y_cm && NY % 8 != 0) || out_stride < NX || out_stride % 4 != 0)
    return VRL_ERR_SHAPE;
  if (NY * (NX / 4) > kMaxGrid * 256LL) return VRL_ERR_SHAPE;
  return VRL_OK;
}

}  // namespace

extern "C" {

int vrl_rowscore(const void* logits, int dtype, int64_t n_rows, int64_t vocab, int64_t row_stride,
                 const int64_t* labels, const float* temperature, float* out_logprob,
                 float* out_entropy, float* out_sum_pi_sq, float* out_lse, int32_t* err_flag,
                 void* stream) {
  const int st = check_rowscore(logits, dtype, n_rows, vocab, row_stride, labels, temperature,
                                out_logprob, out_entropy, out_sum_pi_sq, out_lse, err_flag);
  if (st != VRL_OK || n_rows == 0) return st;
  const RowArgs a{logits, n_rows, vocab, row_stride, labels, temperature, out_logprob, out_entropy,
                  out_sum_pi_sq, out_lse, err_flag, 1, nullptr, static_cast<hipStream_t>(stream)};
  launch_rows_any(dtype, a);
  return launch_status();
}

int vrl_label_logprob(const void* logits, int dtype, int64_t n_rows, int64_t vocab, int64_t row_stride,
                      const int64_t* labels, const float* temperature, const float* lse, float* out_logprob,
                      int32_t* err_flag, void* stream) {
  if (!known_dtype(dtype)) return VRL_ERR_DTYPE;
  if (n_rows < 0 || vocab <= 0 || row_stride < vocab || (n_rows + 255) / 256 > kMaxGrid) return VRL_ERR_SHAPE;
  if (n_rows == 0) return VRL_OK;
  if (logits == nullptr || labels == nullptr || lse == nullptr || out_logprob == nullptr || err_flag == nullptr)
    return VRL_ERR_NULL;
  const uintptr_t esize = (dtype == VRL_F32) ? 4 : 2;
  if (!aligned(logits, esize) || !aligned(labels, 8) || !aligned(temperature, 4) || !aligned(lse, 4) ||
      !aligned(out_logprob, 4) || !aligned(err_flag, 4))
    return VRL_ERR_ALIGN;
  const dim3 grid(static_cast<unsigned>((n_rows + 255) / 256));
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (dtype == VRL_F32) {
    if (temperature != nullptr)
      vrl::label_logprob_kernel<VRL_F32, true><<<grid, dim3(256), 0, s>>>(logits, n_rows, vocab, row_stride, labels,
                                                                          temperature, lse, out_logprob, err_flag);
    else
      vrl::label_logprob_kernel<VRL_F32, false><<<grid, dim3(256), 0, s>>>(logits, n_rows, vocab, row_stride, labels,
                                                                           temperature, lse, out_logprob, err_flag);
  } else if (dtype == VRL_BF16) {
    vrl::label_logprob_kernel<VRL_BF16, false><<<grid, dim3(256), 0, s>>>(logits, n_rows, vocab, row_stride, labels,
                                                                          temperature, lse, out_logprob, err_flag);
  } else {
    vrl::label_logprob_kernel<VRL_F16, false><<<grid, dim3(256), 0, s>>>(logits, n_rows, vocab, row_stride, labels,
                                                                         temperature, lse, out_logprob, err_flag);
  }
  return launch_status();
}

int vrl_score_responses(const void* logits, int dtype, int64_t n_rows, int64_t vocab, int64_t row_stride,
                        const int64_t* labels, const int64_t* input_ids, const float* temperature,
                        const int64_t* cu_seqlens, const int64_t* response_lens, int64_t B, int64_t T_out,
                        float* out_logprob, float* out_entropy, float* resp_logprob, float* resp_entropy,
                        float* resp_lse, int32_t* err_flag, void* stream) {
  if (!known_dtype(dtype)) return VRL_ERR_DTYPE;
  if (n_rows < 0 || vocab <= 0 || row_stride < vocab || B < 0 || T_out < 0 || n_rows + B > kMaxGrid)
    return VRL_ERR_SHAPE;
  if (resp_logprob == nullptr && resp_entropy == nullptr && resp_lse == nullptr) return VRL_ERR_ARG;
  if (labels != nullptr && input_ids != nullptr) return VRL_ERR_ARG;   // one source of labels
  if (out_logprob != nullptr && resp_logprob == nullptr) return VRL_ERR_ARG;
  if (out_entropy != nullptr && resp_entropy == nullptr) return VRL_ERR_ARG;
  if (B == 0) return (n_rows == 0) ? VRL_OK : VRL_ERR_SHAPE;          // rows that belong to no sequence
  if (cu_seqlens == nullptr || response_lens == nullptr || err_flag == nullptr) return VRL_ERR_NULL;
  if (n_rows > 0 && logits == nullptr) return VRL_ERR_NULL;
  if (resp_logprob != nullptr && labels == nullptr && input_ids == nullptr && n_rows > 0) return VRL_ERR_NULL;
  const uintptr_t esize = (dtype == VRL_F32) ? 4 : 2;
  if (!aligned(logits, esize) || !aligned(labels, 8) || !aligned(input_ids, 8) || !aligned(temperature, 4) ||
      !aligned(cu_seqlens, 8) || !aligned(response_lens, 8) || !aligned(out_logprob, 4) ||
      !aligned(out_entropy, 4) || !aligned(resp_logprob, 4) || !aligned(resp_entropy, 4) || !aligned(resp_lse, 4) ||
      !aligned(err_flag, 4))
    return VRL_ERR_ALIGN;
  hipStream_t s = static_cast<hipStream_t>(stream);
#define VRL_SR_ARGS                                                                                               \
  n_rows, vocab, logits, n_rows, vocab, row_stride, labels, input_ids, temperature, cu_seqlens, response_lens, B, \
      T_out, out_logprob, out_entropy, resp_logprob, resp_entropy, resp_lse, err_flag, s
  if (dtype == VRL_F32) {
    if (temperature != nullptr)
      launch_score_responses_shaped<VRL_F32, true>(VRL_SR_ARGS);
    else
      launch_score_responses_shaped<VRL_F32, false>(VRL_SR_ARGS);
  } else if (dtype == VRL_BF16) {
    launch_score_responses_shaped<VRL_BF16, false>(VRL_SR_ARGS);
  } else {
    launch_score_responses_shaped<VRL_F16, false>(VRL_SR_ARGS);
  }
#undef VRL_SR_ARGS
  return launch_status();
}

// The backward walk without rows (rowscore_backward_flat_kernel), for inputs of at least 2^22 vectors (64 MiB; below
// that one workgroup per row is as fast). Many short workgroups beat few long ones: at 8192 x 151936 bf16 512 workgroups
// take 936 us, 4096 922, 16384 883, 32768 885, one per trip (75970) 907, against 949 us for one workgroup per row;
// 2048 x 128256 fp32: 378, 375, 357, 347, 346 against 421 us.
constexpr int64_t kFlatBackwardGrid = 32768;
constexpr int64_t kFlatBackwardMinVecs = int64_t(1) << 22;


// Workgroups for that walk, or 0 when the rows do not lie back to back on 16-byte boundaries, are shorter than a
// wavefront's trip, or are too few.
int64_t flat_backward_grid(const void* logits, const void* dlogits, int64_t n_rows, int64_t vocab, int64_t row_stride,
                           int64_t d_row_stride, int64_t esize) {
  const int64_t per_vec = 16 / esize;
  if (row_stride != vocab || d_row_stride != vocab || vocab % per_vec != 0 ||
      vocab / per_vec < vrl::kFlatBackwardTripVecs || !aligned(logits, 16) || !aligned(dlogits, 16) ||
      n_rows * (vocab / per_vec) < kFlatBackwardMinVecs)
    return 0;
  constexpr int64_t wg_vecs = (vrl::kFlatBackwardThreads / 64) * vrl::kFlatBackwardTripVecs;
  const int64_t trips = (n_rows * (vocab / per_vec) + wg_vecs - 1) / wg_vecs;
  return trips < kFlatBackwardGrid ? trips : kFlatBackwardGrid;
}

int vrl_score_responses_backward(const void* logits, int dtype, int64_t n_rows, int64_t vocab, int64_t row_stride,
                                 const int64_t* labels, const int64_t* input_ids, const float* temperature,
                                 const int64_t* cu_seqlens, const int64_t* response_lens, int64_t B, int64_t T_out,
                                 const float* resp_lse, const float* resp_entropy, const float* g_resp_logprob,
                                 const float* g_resp_entropy, void* dlogits, int64_t d_row_stride, void* stream) {
  if (!known_dtype(dtype)) return VRL_ERR_DTYPE;
  if (n_rows < 0 || vocab <= 0 || row_stride < vocab || d_row_stride < vocab || B < 0 || T_out < 0 ||
      n_rows > kMaxGrid)
    return VRL_ERR_SHAPE;
  if (B == 0 && n_rows > 0) return VRL_ERR_SHAPE;  // rows that belong to no sequence
  if (g_resp_logprob == nullptr && g_resp_entropy == nullptr) return VRL_ERR_ARG;
  if (labels != nullptr && input_ids != nullptr) return VRL_ERR_ARG;
  if (n_rows == 0) return VRL_OK;
  if (logits == nullptr || dlogits == nullptr) return VRL_ERR_NULL;
  if (B > 0 && (cu_seqlens == nullptr || response_lens == nullptr || resp_lse == nullptr)) return VRL_ERR_NULL;
  if (g_resp_logprob != nullptr && labels == nullptr && input_ids == nullptr) return VRL_ERR_NULL;
  if (g_resp_entropy != nullptr && resp_entropy == nullptr && B > 0) return VRL_ERR_NULL;
  const uintptr_t esize = (dtype == VRL_F32) ? 4 : 2;
  if (!aligned(logits, esize) || !aligned(dlogits, esize) || !aligned(labels, 8) || !aligned(input_ids, 8) ||
      !aligned(temperature, 4) || !aligned(cu_seqlens, 8) || !aligned(response_lens, 8) || !aligned(resp_lse, 4) ||
      !aligned(resp_entropy, 4) || !aligned(g_resp_logprob, 4) || !aligned(g_resp_entropy, 4))
    return VRL_ERR_ALIGN;
  hipStream_t s = static_cast<hipStream_t>(stream);
  // few sequences (a wavefront looks a row's sequence up with one ballot) and rows back to back: the walk without rows
  const int64_t flat = B <= 64 ? flat_backward_grid(logits, dlogits, n_rows, vocab, row_stride, d_row_stride,
                                                    static_cast<int64_t>(esize)) : 0;
  if (flat > 0) {
    const dim3 fg(static_cast<unsigned>(flat)), fb(vrl::kFlatBackwardThreads);
#define VRL_SRBF_ARGS                                                                                                 \
  logits, n_rows, vocab, labels, input_ids, temperature, cu_seqlens, response_lens, B, T_out, resp_lse, resp_entropy, \
      g_resp_logprob, g_resp_entropy, dlogits
    if (dtype == VRL_F32)
      vrl::score_responses_backward_flat_kernel<VRL_F32><<<fg, fb, 0, s>>>(VRL_SRBF_ARGS);
    else if (dtype == VRL_BF16)
      vrl::score_responses_backward_flat_kernel<VRL_BF16><<<fg, fb, 0, s>>>(VRL_SRBF_ARGS);
    else
      vrl::score_responses_backward_flat_kernel<VRL_F16><<<fg, fb, 0, s>>>(VRL_SRBF_ARGS);
#undef VRL_SRBF_ARGS
    return launch_status();
  }
  const dim3 grid(static_cast<unsigned>(n_rows));
  const dim3 block(kBackwardWaves * 64);
#define VRL_SRB_ARGS                                                                                                  \
  logits, n_rows, vocab, row_stride, labels, input_ids, temperature, cu_seqlens, response_lens, B, T_out, resp_lse, \
      resp_entropy, g_resp_logprob, g_resp_entropy, dlogits, d_row_stride
  if (dtype == VRL_F32)
    vrl::score_responses_backward_kernel<VRL_F32, kBackwardWaves, kBackwardUnroll><<<grid, block, 0, s>>>(VRL_SRB_ARGS);
  else if (dtype == VRL_BF16)
    vrl::score_responses_backward_kernel<VRL_BF16, kBackwardWaves, kBackwardUnroll><<<grid, block, 0, s>>>(VRL_SRB_ARGS);
  else
    vrl::score_responses_backward_kernel<VRL_F16, kBackwardWaves, kBackwardUnroll><<<grid, block, 0, s>>>(VRL_SRB_ARGS);
#undef VRL_SRB_ARGS
  return launch_status();
}

int vrl_rowscore_split_plan(int dtype, int64_t n_rows, int64_t vocab) {
  if (!known_dtype(dtype) || n_rows <= 0 || vocab <= 0) return 1;
  // A 16-wavefront workgroup per row already keeps a whole CU streaming, so from 128 rows on one
  // workgroup per row is as fast or faster (measured at vocab 151936 bf16: 256 rows 15.1 us against
  // 18.2 us split, 512 rows 26.0 against 29.7; 64 rows 13.2 against 13.0; 8 rows 11.2 against 9.8).
  // Below that, slices of a row spread over idle CUs shorten the one row's latency a little.
  constexpr int64_t kSplitBelowRows = 128;
  constexpr int64_t kTargetGroups = 1024;
  if (n_rows >= kSplitBelowRows) return 1;
  int64_t want = (kTargetGroups + n_rows - 1) / n_rows;
  // every slice keeps at least two register batches of the split workgroup
  const int64_t per_vec = (dtype == VRL_F32) ? 4 : 8;
  const int64_t batch = static_cast<int64_t>(kSplitWaves) * 64 * kSplitUnroll * per_vec;
  const int64_t by_size = vocab / (2 * batch);
  if (want > by_size) want = by_size;
  if (want > kMaxSplits) want = kMaxSplits;
  return want < 2 ? 1 : static_cast<int>(want);
}

int vrl_rowscore_split(const void* logits, int dtype, int64_t n_rows, int64_t vocab, int64_t row_stride,
                       const int64_t* labels, const float* temperature, float* out_logprob,
                       float* out_entropy, float* out_sum_pi_sq, float* out_lse, int32_t* err_flag,
                       int n_splits, float* partials, void* stream) {
  const int st = check_rowscore(logits, dtype, n_rows, vocab, row_stride, labels, temperature,
                                out_logprob, out_entropy, out_sum_pi_sq, out_lse, err_flag);
  if (st != VRL_OK) return st;
  if (n_splits < 1 || n_splits > kMaxSplits) return VRL_ERR_ARG;
  if (n_rows * n_splits > kMaxGrid) return VRL_ERR_SHAPE;
  if (n_rows == 0) return VRL_OK;
  if (n_splits > 1 && partials == nullptr) return VRL_ERR_NULL;
  if (!aligned(partials, 4)) return VRL_ERR_ALIGN;
  const RowArgs a{logits, n_rows, vocab, row_stride, labels, temperature, out_logprob, out_entropy,
                  out_sum_pi_sq, out_lse, err_flag, n_splits, partials, static_cast<hipStream_t>(stream)};
  launch_rows_any(dtype, a);
  return launch_status();
}

int vrl_rowscore_split_static(const void* logits, int dtype, int64_t n_rows, int64_t vocab, int64_t row_stride,
                              const int64_t* labels, const float* temperature, float* out_logprob,
                              float* out_entropy, float* out_sum_pi_sq, float* out_lse, int32_t* err_flag,
                              int n_splits, void* stream) {
  const int st = check_rowscore(logits, dtype, n_rows, vocab, row_stride, labels, temperature,
                                out_logprob, out_entropy, out_sum_pi_sq, out_lse, err_flag);
  if (st != VRL_OK) return st;
  if (n_splits < 1 || n_splits > kMaxSplits) return VRL_ERR_ARG;
  if (n_rows * n_splits > kMaxGrid) return VRL_ERR_SHAPE;
  if (n_splits > 1 && n_rows * n_splits > VRL_STATIC_PARTIALS_MAX) return VRL_ERR_SCRATCH;
  if (n_rows == 0) return VRL_OK;
  float* partials = nullptr;
  if (n_splits > 1) {
    const int ss = static_scratch(&partials);
    if (ss != VRL_OK) return ss;
  }
  // Every (row, slice) partial the merge kernel reads is written by the split kernel of the same call first, so
  // nothing in the array has to start at zero.
  const RowArgs a{logits, n_rows, vocab, row_stride, labels, temperature, out_logprob, out_entropy,
                  out_sum_pi_sq, out_lse, err_flag, n_splits, partials, static_cast<hipStream_t>(stream)};
  launch_rows_any(dtype, a);
  return launch_status();
}

int vrl_rowscore_backward(const void* logits, int dtype, int64_t n_rows, int64_t vocab, int64_t row_stride,
                          const int64_t* labels, const float* temperature, const float* lse,
                          const float* entropy, const float* g_logprob, const float* g_entropy,
                          void* dlogits, int64_t d_row_stride, void* stream) {
  if (!known_dtype(dtype)) return VRL_ERR_DTYPE;
  if (n_rows < 0 || vocab <= 0 || row_stride < vocab || d_row_stride < vocab || n_rows > kMaxGrid)
    return VRL_ERR_SHAPE;
  if (g_logprob == nullptr && g_entropy == nullptr) return VRL_ERR_ARG;
  if (n_rows == 0) return VRL_OK;
  if (logits == nullptr || dlogits == nullptr || lse == nullptr) return VRL_ERR_NULL;
  if (g_logprob != nullptr && labels == nullptr) return VRL_ERR_NULL;
  if (g_entropy != nullptr && entropy == nullptr) return VRL_ERR_NULL;
  const uintptr_t esize = (dtype == VRL_F32) ? 4 : 2;
  if (!aligned(logits, esize) || !aligned(dlogits, esize) || !aligned(labels, 8) || !aligned(temperature, 4) ||
      !aligned(lse, 4) || !aligned(entropy, 4) || !aligned(g_logprob, 4) || !aligned(g_entropy, 4))
    return VRL_ERR_ALIGN;
  const dim3 grid(static_cast<unsigned>(n_rows));
  hipStream_t s = static_cast<hipStream_t>(stream);
  // Rows that lie back to back on 16-byte boundaries, enough of them: the walk without rows.
  const int64_t flat = flat_backward_grid(logits, dlogits, n_rows, vocab, row_stride, d_row_stride, static_cast<int64_t>(esize));
  if (flat > 0) {
    const dim3 fg(static_cast<unsigned>(flat)), fb(vrl::kFlatBackwardThreads);
    if (dtype == VRL_F32)
      vrl::rowscore_backward_flat_kernel<VRL_F32><<<fg, fb, 0, s>>>(logits, n_rows, vocab, labels, temperature, lse, entropy,
                                                                   g_logprob, g_entropy, dlogits);
    else if (dtype == VRL_BF16)
      vrl::rowscore_backward_flat_kernel<VRL_BF16><<<fg, fb, 0, s>>>(logits, n_rows, vocab, labels, temperature, lse, entropy,
                                                                    g_logprob, g_entropy, dlogits);
    else
      vrl::rowscore_backward_flat_kernel<VRL_F16><<<fg, fb, 0, s>>>(logits, n_rows, vocab, labels, temperature, lse, entropy,
                                                                   g_logprob, g_entropy, dlogits);
    return launch_status();
  }
  if (dtype == VRL_F32)
    vrl::rowscore_backward_kernel<VRL_F32, kBackwardWaves, kBackwardUnroll><<<grid, dim3(kBackwardWaves * 64), 0, s>>>(
        logits, vocab, row_stride, labels, temperature, lse, entropy, g_logprob, g_entropy, dlogits, d_row_stride);
  else if (dtype == VRL_BF16)
    vrl::rowscore_backward_kernel<VRL_BF16, kBackwardWaves, kBackwardUnroll><<<grid, dim3(kBackwardWaves * 64), 0, s>>>(
        logits, vocab, row_stride, labels, temperature, lse, entropy, g_logprob, g_entropy, dlogits, d_row_stride);
  else
    vrl::rowscore_backward_kernel<VRL_F16, kBackwardWaves, kBackwardUnroll><<<grid, dim3(kBackwardWaves * 64), 0, s>>>(
        logits, vocab, row_stride, labels, temperature, lse, entropy, g_logprob, g_entropy, dlogits, d_row_stride);
  return launch_status();
}

int vrl_rollout_corr(const float* old_log_prob, const float* rollout_log_prob, const uint8_t* mask, int64_t B,
                     int64_t T, int is_mode, int icepop, float is_upper, float is_lower, float is_lower_metric,
                     uint32_t rs_bits, const float* rs_lo_host, const float* rs_hi_host, float* weights,
                     uint8_t* keep, float* stats, int32_t* seq_keep_bits, void* stream) {
  if (B < 0 || T < 0 || B > kMaxGrid || T > kMaxGrid) return VRL_ERR_SHAPE;
  if (is_mode < 0 || is_mode > 2 || (rs_bits >> vrl::kNumRsOptions) != 0) return VRL_ERR_ARG;
  if (rs_bits != 0 && (rs_lo_host == nullptr || rs_hi_host == nullptr)) return VRL_ERR_NULL;
  if (B == 0) return VRL_OK;
  if (stats == nullptr || seq_keep_bits == nullptr) return VRL_ERR_NULL;
  if (T > 0 && (old_log_prob == nullptr || rollout_log_prob == nullptr)) return VRL_ERR_NULL;
  if (!aligned(old_log_prob, 4) || !aligned(rollout_log_prob, 4) || !aligned(weights, 4) || !aligned(stats, 4) ||
      !aligned(seq_keep_bits, 4))
    return VRL_ERR_ALIGN;
  vrl::CorrCfg cfg;
  cfg.is_mode = is_mode;
  cfg.icepop = icepop ? 1 : 0;
  cfg.is_upper = is_upper;
  cfg.is_lower = is_lower;
  cfg.is_lower_metric = is_lower_metric;
  cfg.rs_bits = rs_bits;
  for (int i = 0; i < vrl::kNumRsOptions; ++i) {
    cfg.rs_lo[i] = (rs_bits != 0) ? rs_lo_host[i] : 0.f;
    cfg.rs_hi[i] = (rs_bits != 0) ? rs_hi_host[i] : 0.f;
  }
  vrl::rollout_corr_kernel<4><<<dim3(static_cast<unsigned>(B)), dim3(256), 0, static_cast<hipStream_t>(stream)>>>(
      old_log_prob, rollout_log_prob, mask, T, cfg, weights, keep, stats, seq_keep_bits);
  return launch_status();
}

int vrl_rollout_corr_num_stats(void) { return vrl::kNumCorrStats; }

int vrl_response_slice(const void* values, int64_t row_bytes, const int64_t* cu_seqlens, const int64_t* response_lens,
                       int64_t B, int64_t n_tokens, int64_t T_out, void* out, int32_t* err_flag, void* stream) {
  if (B < 0 || T_out < 0 || n_tokens < 0 || B > kMaxGrid || row_bytes <= 0 || row_bytes > kMaxRowBytes)
    return VRL_ERR_SHAPE;
  if (B == 0 || T_out == 0) return VRL_OK;
  if ((values == nullptr && n_tokens > 0) || cu_seqlens == nullptr || response_lens == nullptr || out == nullptr ||
      err_flag == nullptr)
    return VRL_ERR_NULL;
  if (!aligned(cu_seqlens, 8) || !aligned(response_lens, 8) || !aligned(err_flag, 4)) return VRL_ERR_ALIGN;
  const int unit = copy_unit(row_bytes, values, out);
  const int64_t row_units = row_bytes / unit;
  if (T_out > (int64_t(1) << 62) / row_units) return VRL_ERR_SHAPE;
  const int64_t chunks = (T_out * row_units + vrl::kSliceChunk - 1) / vrl::kSliceChunk;
  if (chunks > kMaxGridY) return VRL_ERR_SHAPE;
  const dim3 grid(static_cast<unsigned>(B), static_cast<unsigned>(chunks));
  hipStream_t s = static_cast<hipStream_t>(stream);
  const char* v = static_cast<const char*>(values);
  char* o = static_cast<char*>(out);
#define VRL_SLICE(U)                                                                                                   \
  vrl::response_slice_kernel<U><<<grid, dim3(vrl::kSliceThreads), 0, s>>>(v, row_units, cu_seqlens, response_lens,     \
                                                                          n_tokens, T_out, o, err_flag)
  switch (unit) {
    case 16: VRL_SLICE(16); break;
    case 8: VRL_SLICE(8); break;
    case 4: VRL_SLICE(4); break;
    case 2: VRL_SLICE(2); break;
    default: VRL_SLICE(1); break;
  }
#undef VRL_SLICE
  return launch_status();
}

int vrl_expand_per_sequence(const float* values, const int64_t* cu_seqlens, int64_t B, int64_t n_tokens, float* out,
                            int32_t* err_flag, void* stream) {
  if (B < 0 || n_tokens < 0 || B > kMaxGrid) return VRL_ERR_SHAPE;
  if (B == 0) return n_tokens == 0 ? VRL_OK : VRL_ERR_SHAPE;   // tokens, but no sequence to take a value from
  if (values == nullptr || cu_seqlens == nullptr || err_flag == nullptr || (out == nullptr && n_tokens > 0))
    return VRL_ERR_NULL;
  if (!aligned(values, 4) || !aligned(out, 4) || !aligned(cu_seqlens, 8) || !aligned(err_flag, 4)) return VRL_ERR_ALIGN;
  const int64_t threads = n_tokens > B + 1 ? n_tokens : B + 1;
  const int64_t blocks = (threads + vrl::kSliceThreads - 1) / vrl::kSliceThreads;
  if (blocks > kMaxGrid) return VRL_ERR_SHAPE;
  vrl::expand_per_sequence_kernel<<<dim3(static_cast<unsigned>(blocks)), dim3(vrl::kSliceThreads), 0,
                                    static_cast<hipStream_t>(stream)>>>(values, cu_seqlens, B, n_tokens, out, err_flag);
  return launch_status();
}

int vrl_response_pack(const void* values, int64_t row_bytes, const int64_t* cu_seqlens, const int64_t* response_lens,
                      const int64_t* out_offsets, int64_t B, int64_t n_tokens, int64_t out_total, void* out,
                      int32_t* err_flag, void* stream) {
  if (B < 0 || out_total < 0 || n_tokens < 0 || B > kMaxGrid || row_bytes <= 0 || row_bytes > kMaxRowBytes)
    return VRL_ERR_SHAPE;
  if (B == 0) return VRL_OK;
  if ((values == nullptr && n_tokens > 0) || cu_seqlens == nullptr || response_lens == nullptr || out_offsets == nullptr ||
      err_flag == nullptr || (out == nullptr && out_total > 0))
    return VRL_ERR_NULL;
  if (!aligned(cu_seqlens, 8) || !aligned(response_lens, 8) || !aligned(out_offsets, 8) || !aligned(err_flag, 4))
    return VRL_ERR_ALIGN;
  const int unit = copy_unit(row_bytes, values, out);
  const int64_t row_units = row_bytes / unit;
  // a window cannot be longer than the shorter of the two arrays; more workgroups per sequence than that needs are idle
  const int64_t longest = out_total < n_tokens ? out_total : n_tokens;
  if (longest > (int64_t(1) << 62) / row_units) return VRL_ERR_SHAPE;
  int64_t chunks = (longest * row_units + vrl::kSliceChunk - 1) / vrl::kSliceChunk;
  if (chunks < 1) chunks = 1;
  if (chunks > kPackMaxChunks) chunks = kPackMaxChunks;   // the kernel strides over what is left
  const dim3 grid(static_cast<unsigned>(B), static_cast<unsigned>(chunks));
  hipStream_t s = static_cast<hipStream_t>(stream);
  const char* v = static_cast<const char*>(values);
  char* o = static_cast<char*>(out);
#define VRL_PACK(U)                                                                                                    \
  vrl::response_pack_kernel<U><<<grid, dim3(vrl::kSliceThreads), 0, s>>>(v, row_units, cu_seqlens, response_lens,      \
                                                                         out_offsets, n_tokens, out_total, o, err_flag)
  switch (unit) {
    case 16: VRL_PACK(16); break;
    case 8: VRL_PACK(8); break;
    case 4: VRL_PACK(4); break;
    case 2: VRL_PACK(2); break;
    default: VRL_PACK(1); break;
  }
#undef VRL_PACK
  return launch_status();
}

int vrl_lmhead_plan(int64_t n_tokens, int64_t vocab) {
  if (n_tokens <= 0 || vocab <= 0) return 1;
  const int64_t tblocks = (n_tokens + vrl::kLmTokens - 1) / vrl::kLmTokens;
  const int64_t vtiles = (vocab + vrl::kLmVocab - 1) / vrl::kLmVocab;
  const int64_t runs = (vtiles + vrl::kLmSubTiles - 1) / vrl::kLmSubTiles;
  const int64_t cus = device_cus();
  // One workgroup per CU runs at a time, so a launch takes (rounds of workgroups) x (tiles of the longest share, plus
  // about half a tile to start a workgroup and fill and drain its ring; with two tiles the choices at 12288 and 20000
  // tokens were 8 % and 4 % slower than what this picks). The fewest splits among the cheapest: a token's results do
  // not depend on the choice (see kLmSubTiles), only the time does.
  int64_t best = 1, best_cost = -1;
  for (int64_t s = 1; s <= vrl::kLmMaxSplits && s <= runs; ++s) {
    const int64_t share = (runs + s - 1) / s;
    if ((runs + share - 1) / share != s) continue;   // this many splits would leave one without a tile
    const int64_t rounds = (tblocks * s + cus - 1) / cus;
    const int64_t cost = rounds * (2 * share * vrl::kLmSubTiles + 1);   // in half tiles
    if (best_cost < 0 || cost < best_cost) {
      best = s;
      best_cost = cost;
    }
  }
  return static_cast<int>(best);
}

int64_t vrl_lmhead_partials(int64_t n_tokens, int64_t vocab) {
  if (n_tokens <= 0 || vocab <= 0) return 0;
  const int64_t vtiles = (vocab + vrl::kLmVocab - 1) / vrl::kLmVocab;
  const int64_t runs = (vtiles + vrl::kLmSubTiles - 1) / vrl::kLmSubTiles;
  return runs * 4 * 3 * n_tokens;   // per token: a (max, sum, weighted sum) state per run and wavefront quarter
}

int vrl_lmhead_score(const void* hidden, const void* weight, int dtype, int64_t n_tokens, int64_t vocab,
                     int64_t hidden_size, int64_t h_stride, int64_t w_stride, const int64_t* labels,
                     const float* temperature, int n_splits, float* partials, float* out_logprob,
                     float* out_entropy, float* out_lse, int32_t* err_flag, void* logits_out, int64_t logits_stride,
                     int64_t logits_rows, void* stream) {
  const int cs = check_lmhead_shape(dtype, n_tokens, vocab, hidden_size, h_stride, w_stride, n_splits);
  if (cs != VRL_OK) return cs;
  if (out_logprob == nullptr && out_entropy == nullptr && out_lse == nullptr && logits_out == nullptr) return VRL_ERR_ARG;
  if (logits_out != nullptr && (logits_rows < 1 || logits_rows > n_tokens)) return VRL_ERR_SHAPE;
  if (hidden == nullptr || weight == nullptr || partials == nullptr) return VRL_ERR_NULL;
  if (out_logprob != nullptr && (labels == nullptr || err_flag == nullptr)) return VRL_ERR_NULL;
  // kept logits: 8-byte stores of 4 consecutive vocabulary entries, so the vocabulary and the pitch must keep them aligned
  if (logits_out != nullptr && (vocab % 8 != 0 || logits_stride < vocab || logits_stride % 8 != 0 || logits_stride > kLmMaxStride))
    return VRL_ERR_SHAPE;
  if (!aligned(hidden, 16) || !aligned(weight, 16) || !aligned(labels, 8) || !aligned(temperature, 4) ||
      !aligned(partials, 4) || !aligned(out_logprob, 4) || !aligned(out_entropy, 4) || !aligned(out_lse, 4) ||
      !aligned(err_flag, 4) || !aligned(logits_out, 16))
    return VRL_ERR_ALIGN;
  hipStream_t s = static_cast<hipStream_t>(stream);
#define VRL_LMHEAD_ARGS                                                                                            \
  hidden, weight, n_tokens, vocab, hidden_size, h_stride, w_stride, labels, temperature, n_splits, partials,        \
      out_logprob, out_entropy, out_lse, err_flag, logits_out, logits_stride, logits_rows, s
  if (dtype == VRL_BF16)
    return logits_out != nullptr ? launch_lmhead<VRL_BF16, true>(VRL_LMHEAD_ARGS) : launch_lmhead<VRL_BF16, false>(VRL_LMHEAD_ARGS);
  return logits_out != nullptr ? launch_lmhead<VRL_F16, true>(VRL_LMHEAD_ARGS) : launch_lmhead<VRL_F16, false>(VRL_LMHEAD_ARGS);
#undef VRL_LMHEAD_ARGS
}

int vrl_lmhead_dlogits(const void* hidden, const void* weight, int dtype, int64_t n_tokens, int64_t vocab,
                       int64_t hidden_size, int64_t h_stride, int64_t w_stride, const int64_t* labels,
                       const float* temperature, const float* lse, const float* entropy, const float* g_logprob,
                       const float* g_entropy, int n_splits, void* dlogits, int64_t d_stride, void* stream) {
  const int cs = check_lmhead_shape(dtype, n_tokens, vocab, hidden_size, h_stride, w_stride, n_splits);
  if (cs != VRL_OK) return cs;
  // 8-byte stores of 4 consecutive vocabulary entries: the vocabulary and the output pitch must keep them aligned
  if (vocab % 8 != 0 || d_stride < vocab || d_stride % 8 != 0) return VRL_ERR_SHAPE;
  if (g_logprob == nullptr && g_entropy == nullptr) return VRL_ERR_ARG;
  if (hidden == nullptr || weight == nullptr || lse == nullptr || dlogits == nullptr) return VRL_ERR_NULL;
  if (g_logprob != nullptr && labels == nullptr) return VRL_ERR_NULL;
  if (g_entropy != nullptr && entropy == nullptr) return VRL_ERR_NULL;
  if (!aligned(hidden, 16) || !aligned(weight, 16) || !aligned(dlogits, 16) || !aligned(labels, 8) ||
      !aligned(temperature, 4) || !aligned(lse, 4) || !aligned(entropy, 4) || !aligned(g_logprob, 4) ||
      !aligned(g_entropy, 4))
    return VRL_ERR_ALIGN;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (dtype == VRL_BF16)
    return launch_lmhead_dlogits<VRL_BF16>(hidden, weight, n_tokens, vocab, hidden_size, h_stride, w_stride, labels,
                                           temperature, lse, entropy, g_logprob, g_entropy, n_splits, dlogits, d_stride,
                                           s);
  return launch_lmhead_dlogits<VRL_F16>(hidden, weight, n_tokens, vocab, hidden_size, h_stride, w_stride, labels,
                                        temperature, lse, entropy, g_logprob, g_entropy, n_splits, dlogits, d_stride, s);
}

int vrl_gemm_nt_plan(int dtype, int64_t NX, int64_t NY, int64_t K, int64_t* workspace_floats) {
  const int st = check_gemm(dtype, NX, NY, K, K, K, 0, 0, NX);
  if (st != VRL_OK) return st;
  const GemmPlan p = gemm_plan(NX, NY, K, 0);
  if (workspace_floats != nullptr) *workspace_floats = p.shape.k_parts > 1 ? p.shape.k_parts * NX * NY : 0;
  return p.shape.k_parts;
}

int vrl_gemm(const void* x, const void* y, int dtype, int64_t NX, int64_t NY, int64_t K, int64_t x_stride,
             int64_t y_stride, int x_contraction_major, int y_contraction_major, void* out, int64_t out_stride,
             int accumulate, int k_parts, float* workspace, void* stream) {
  const int x_cm = x_contraction_major != 0, y_cm = y_contraction_major != 0;
  const int st = check_gemm(dtype, NX, NY, K, x_stride, y_stride, x_cm, y_cm, out_stride);
  if (st != VRL_OK) return st;
  if (k_parts < 1 || k_parts > 16 || K / vrl::kLmK / k_parts < 2) return VRL_ERR_ARG;
  if (x == nullptr || y == nullptr || out == nullptr) return VRL_ERR_NULL;
  const GemmPlan p = gemm_plan(NX, NY, K, k_parts);
  if (p.shape.k_parts > 1 && workspace == nullptr) return VRL_ERR_NULL;
  if (!aligned(x, 16) || !aligned(y, 16) || !aligned(out, 8) || !aligned(workspace, 16)) return VRL_ERR_ALIGN;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (dtype == VRL_BF16)
    return launch_gemm_layout<VRL_BF16>(x_cm, y_cm, x, y, p, x_stride, y_stride, out, out_stride, accumulate, workspace,
                                        s);
  return launch_gemm_layout<VRL_F16>(x_cm, y_cm, x, y, p, x_stride, y_stride, out, out_stride, accumulate, workspace, s);
}

int vrl_gemm_nt(const void* x, const void* y, int dtype, int64_t NX, int64_t NY, int64_t K, int64_t x_stride,
                int64_t y_stride, void* out, int64_t out_stride, int accumulate, int k_parts, float* workspace,
                void* stream) {
  return vrl_gemm(x, y, dtype, NX, NY, K, x_stride, y_stride, 0, 0, out, out_stride, accumulate, k_parts, workspace,
                  stream);
}

int vrl_transpose(const void* src, int elem_size, int64_t rows, int64_t cols, int64_t src_stride,
                  void* dst, int64_t dst_stride, void* stream) {
  if (elem_size != 2 && elem_size != 4) return VRL_ERR_DTYPE;
  if (rows < 0 || cols < 0 || src_stride < cols || dst_stride < rows) return VRL_ERR_SHAPE;
  if (rows == 0 || cols == 0) return VRL_OK;
  if (src == nullptr || dst == nullptr) return VRL_ERR_NULL;
  if (!aligned(src, elem_size) || !aligned(dst, elem_size)) return VRL_ERR_ALIGN;
  {  // the two arrays must not share a byte
    const char* s0 = static_cast<const char*>(src);
    const char* s1 = s0 + ((rows - 1) * src_stride + cols) * elem_size;
    const char* d0 = static_cast<const char*>(dst);
    const char* d1 = d0 + ((cols - 1) * dst_stride + rows) * elem_size;
    if (s0 < d1 && d0 < s1) return VRL_ERR_ARG;
  }
  const int tile = elem_size == 2 ? vrl::TransposeShape<2>::kTile : vrl::TransposeShape<4>::kTile;
  const int64_t tiles_r = (rows + tile - 1) / tile;
  const int64_t tiles_c = (cols + tile - 1) / tile;
  if (tiles_r * tiles_c > kMaxGrid) return VRL_ERR_SHAPE;
  const int vec_ok = aligned(src, 16) && aligned(dst, 16) && (src_stride * elem_size) % 16 == 0 &&
                     (dst_stride * elem_size) % 16 == 0;
  const dim3 grid(static_cast<unsigned>(tiles_r * tiles_c));
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (elem_size == 2) {
    vrl::transpose_kernel<2><<<grid, dim3(256), 0, s>>>(static_cast<const char*>(src), rows, cols, src_stride,
                                                        static_cast<char*>(dst), dst_stride, tiles_c, vec_ok);
  } else {
    vrl::transpose_kernel<4><<<grid, dim3(256), 0, s>>>(static_cast<const char*>(src), rows, cols, src_stride,
                                                        static_cast<char*>(dst), dst_stride, tiles_c, vec_ok);
  }
  return launch_status();
}

int64_t vrl_spec_verify_workspace(int64_t n_tokens) {
  return n_tokens > 0 ? vrl::flat_workspace_bytes(n_tokens) : 0;
}

int vrl_spec_verify_plan(int packed, int64_t B, int64_t T, int64_t n_tokens) {
  if (B <= 0 || n_tokens < kFlatMinTokens) return 0;
  // Packed lengths live on the device: from this many tokens on, one long sequence among them would cost a workgroup
  // per sequence more than the second launch costs. Padded: few long sequences leave most CUs without a workgroup.
  if (packed) return 1;
  return (T >= kFlatMinPaddedT && B < 2 * device_cus()) ? 1 : 0;
}

int vrl_spec_verify(const float* logp_new, const float* logp_old, const float* log_u,
                    const uint8_t* mask, const int64_t* cu_seqlens, int64_t B, int64_t T, int64_t n_tokens,
                    float thresh_offset, float near_eps, uint8_t* accept, int32_t* first_reject,
                    int32_t* prefix_len, int32_t* near_count, const int64_t* draft_ids,
                    int64_t pad_id, int64_t* out_ids, uint8_t* out_mask, int32_t* err_flag, void* workspace,
                    int64_t workspace_bytes, void* stream) {
  const int st = check_verify(logp_new, logp_old, log_u, mask, cu_seqlens, B, T, n_tokens, err_flag, accept,
                              first_reject, prefix_len, near_count, draft_ids, out_ids, out_mask);
  if (st != VRL_OK || B == 0) return st;
  if (workspace_bytes < 0 || (workspace == nullptr && workspace_bytes != 0)) return VRL_ERR_ARG;
  if (workspace != nullptr && workspace_bytes < vrl_spec_verify_workspace(n_tokens)) return VRL_ERR_SHAPE;
  if (!aligned(workspace, 8)) return VRL_ERR_ALIGN;
  const vrl::VerifyArgs v{logp_new, logp_old, log_u, mask, cu_seqlens, B, T, n_tokens, err_flag, thresh_offset,
                          near_eps, accept, first_reject, prefix_len, near_count, draft_ids, pad_id, out_ids,
                          out_mask};
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (workspace != nullptr && n_tokens > 0) {
    // two flat passes over the tokens (verify_flat_kernels.h): a workspace is the caller's request for them
    const vrl::FlatWork ws = vrl::flat_work(workspace, n_tokens);
    const int64_t draft_tiles = out_ids != nullptr ? ws.n_tiles : 0;
    const int64_t finish_grid = draft_tiles + (B + 3) / 4;
    if (ws.n_tiles > kMaxGrid || finish_grid > kMaxGrid) return VRL_ERR_SHAPE;
    vrl::verify_tokens_kernel<<<dim3(static_cast<unsigned>(ws.n_tiles)), dim3(vrl::kFlatThreads), 0, s>>>(v, ws);
    vrl::verify_finish_kernel<<<dim3(static_cast<unsigned>(finish_grid)), dim3(vrl::kFlatThreads), 0, s>>>(v, ws,
                                                                                                         draft_tiles);
    return launch_status();
  }
  const dim3 grid(static_cast<unsigned>(B));
  // 16-byte accesses when every array allows them (what an allocator hands out does; a view that starts at an odd
  // element may not): same results, fewer and wider memory instructions.
  const bool vec = aligned(logp_new, 16) && aligned(logp_old, 16) && aligned(log_u, 16) && aligned(mask, 4) &&
                   aligned(accept, 4) && aligned(draft_ids, 16) && aligned(out_ids, 16) && aligned(out_mask, 4);
  const int waves = verify_waves(cu_seqlens, B, T);
  if (vec) {
    switch (waves) {
      case 1: vrl::spec_verify_vec_kernel<1><<<grid, dim3(64), 0, s>>>(v); break;
      case 4: vrl::spec_verify_vec_kernel<4><<<grid, dim3(256), 0, s>>>(v); break;
      default: vrl::spec_verify_vec_kernel<16><<<grid, dim3(1024), 0, s>>>(v); break;
    }
  } else {
    switch (waves) {
      case 1: vrl::spec_verify_kernel<1><<<grid, dim3(64), 0, s>>>(v); break;
      case 4: vrl::spec_verify_kernel<4><<<grid, dim3(256), 0, s>>>(v); break;
      default: vrl::spec_verify_kernel<16><<<grid, dim3(1024), 0, s>>>(v); break;
    }
  }
  return launch_status();
}

int vrl_truncate_draft(const int64_t* draft_ids, const uint8_t* mask, const int64_t* cu_seqlens,
                       int64_t B, int64_t T, int64_t n_tokens, const int32_t* first_reject, int64_t pad_id,
                       int64_t* out_ids, uint8_t* out_mask, int32_t* err_flag, void* stream) {
  const int ls = check_layout(cu_seqlens, B, T, n_tokens, err_flag);
  if (ls != VRL_OK) return ls;
  if (B == 0 || n_tokens == 0) return VRL_OK;
  if (draft_ids == nullptr || first_reject == nullptr || out_ids == nullptr || out_mask == nullptr)
    return VRL_ERR_NULL;
  if (!aligned(draft_ids, 8) || !aligned(out_ids, 8) || !aligned(first_reject, 4)) return VRL_ERR_ALIGN;
  const dim3 grid(static_cast<unsigned>(B));
  hipStream_t s = static_cast<hipStream_t>(stream);
  switch (verify_waves(cu_seqlens, B, T)) {
    case 1: vrl::truncate_draft_kernel<1><<<grid, dim3(64), 0, s>>>(draft_ids, mask, cu_seqlens, T, n_tokens, first_reject, pad_id, out_ids, out_mask, err_flag); break;
    case 4: vrl::truncate_draft_kernel<4><<<grid, dim3(256), 0, s>>>(draft_ids, mask, cu_seqlens, T, n_tokens, first_reject, pad_id, out_ids, out_mask, err_flag); break;
    default: vrl::truncate_draft_kernel<16><<<grid, dim3(1024), 0, s>>>(draft_ids, mask, cu_seqlens, T, n_tokens, first_reject, pad_id, out_ids, out_mask, err_flag); break;
  }
  return launch_status();
}

int vrl_fused_score_verify(const void* logits, int dtype, int64_t n_rows, int64_t vocab,
                           int64_t row_stride, const int64_t* labels, const float* temperature,
                           float* out_logprob, float* out_entropy, float* out_sum_pi_sq, float* out_lse,
                           int32_t* err_flag, const float* logp_old, const float* log_u, const uint8_t* mask,
                           const int64_t* cu_seqlens, int64_t B, int64_t T, float thresh_offset,
                           float near_eps, uint8_t* accept, int32_t* first_reject,
                           int32_t* prefix_len, int32_t* near_count, const int64_t* draft_ids,
                           int64_t pad_id, int64_t* out_ids, uint8_t* out_mask, void* stream) {
  // Check both halves before anything is enqueued.
  if (out_logprob == nullptr && n_rows > 0) return VRL_ERR_NULL;
  int st = check_rowscore(logits, dtype, n_rows, vocab, row_stride, labels, temperature, out_logprob,
                          out_entropy, out_sum_pi_sq, out_lse, err_flag);
  if (st != VRL_OK) return st;
  // the row space is the token space: n_rows is what the packed offsets are held to
  st = check_verify(out_logprob, logp_old, log_u, mask, cu_seqlens, B, T, n_rows, err_flag, accept, first_reject,
                    prefix_len, near_count, draft_ids, out_ids, out_mask);
  if (st != VRL_OK) return st;
  st = vrl_rowscore(logits, dtype, n_rows, vocab, row_stride, labels, temperature, out_logprob,
                    out_entropy, out_sum_pi_sq, out_lse, err_flag, stream);
  if (st != VRL_OK) return st;
  return vrl_spec_verify(out_logprob, logp_old, log_u, mask, cu_seqlens, B, T, n_rows, thresh_offset, near_eps,
                         accept, first_reject, prefix_len, near_count, draft_ids, pad_id, out_ids,
                         out_mask, err_flag, nullptr, 0, stream);
}

const char* vrl_strerror(int status) {
  switch (status) {
    case VRL_OK: return "ok";
    case VRL_ERR_NULL: return "a required pointer is NULL";
    case VRL_ERR_DTYPE: return "unsupported logits dtype (expected VRL_F32, VRL_BF16 or VRL_F16)";
    case VRL_ERR_SHAPE: return "bad shape (negative count, vocab <= 0, row_stride < vocab, or too many rows)";
    case VRL_ERR_ALIGN: return "pointer is not aligned to its element size";
    case VRL_ERR_HIP: return "the HIP runtime refused the kernel launch";
    case VRL_ERR_ARG: return "inconsistent optional arguments";
    case VRL_ERR_SCRATCH:
      return "n_rows * n_splits exceeds VRL_STATIC_PARTIALS_MAX, the size of the library's static scratch";
    default: return "unknown vrl status";
  }
}

const char* vrl_last_hip_error(void) { return g_hip_error; }

int vrl_abi_version(void) { return VRL_ABI_VERSION; }

}  // extern "C"
