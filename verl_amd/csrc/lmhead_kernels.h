// LM head fused with the row reduction: logits[tok][v] = sum_k H[tok][k] * W[v][k] are formed on the matrix cores
// and folded straight into the online-softmax partial (m, s, t) of their token; they never reach HBM.
//
// lmhead_partial_kernel: one workgroup of 8 wavefronts (two per SIMD) owns 256 tokens and walks a range of 256-row
// vocabulary tiles (its "split"); per tile it runs the full contraction in steps of 64 (v_mfma_f32_32x32x16 on
// bf16 / fp16, fp32 accumulators). A wavefront owns a 64 (vocabulary) x 128 (tokens) part of the tile: 8 blocks of
// 32x32 = 128 accumulator registers, so two wavefronts fit a SIMD and one's matrix instructions cover the other's
// waits. Operands go global -> LDS directly (128-bit loads, two 64 KiB stages = 128 KiB of LDS, one workgroup per CU),
// swizzled so that the 128-bit fragment reads are free of bank conflicts (measured: SQ_LDS_BANK_CONFLICT = 0).
// A step is four quarter steps of 16 contraction elements. The workgroup barrier sits before the LAST quarter's matrix
// instructions: that quarter's fragments are already in registers, so behind the barrier the first fragments of the
// next step are fetched and the loads of the step after are issued while the matrix cores still work on this step.
// The MFMA is issued with the vocabulary on its row side so that a lane's 16 results of a block belong to ONE
// token: the softmax state needs no cross-lane traffic until the very end.
//
// lmhead_finish_kernel: one wavefront per token forms the label's logit as a dot product in fp32, merges the
// token's partials over the splits and writes log-prob, entropy and logsumexp (same finish as the row kernel).
//
// Roofline: dense bf16 MFMA. 2 * tokens * vocab * hidden flops; HBM traffic is the weight once per XCD group.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "rowscore_kernels.h"

namespace vrl {

#define VRL_LDS_AS __attribute__((address_space(3)))
#define VRL_GLOBAL_AS __attribute__((address_space(1)))

typedef float lm_f32x16 __attribute__((ext_vector_type(16)));

constexpr int kLmTokens = 256;                    // tokens per workgroup tile
constexpr int kLmVocab = 256;                     // vocabulary rows per tile
constexpr int kLmK = 64;                          // contraction elements per step: 128 bytes per tile row, whole cache lines
constexpr int kLmRowBytes = kLmK * 2;
constexpr int kLmTileBytes = 256 * kLmRowBytes;   // one operand tile in LDS (32 KiB)
constexpr int kLmLdsBytes = 4 * kLmTileBytes;     // two stages of (W tile, H tile)
constexpr int kLmMaxSplits = 64;

template <int DT>
struct LmFrag;
template <>
struct LmFrag<1> {
  typedef __bf16 type __attribute__((ext_vector_type(8)));
  __device__ static __forceinline__ lm_f32x16 mfma(type a, type b, lm_f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
  }
};
template <>
struct LmFrag<2> {
  typedef _Float16 type __attribute__((ext_vector_type(8)));
  __device__ static __forceinline__ lm_f32x16 mfma(type a, type b, lm_f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
  }
};

constexpr int kLmWaves = 8;                       // wavefronts per workgroup: 4 vocabulary quarters x 2 token halves

// One wave instruction moves 8 tile rows x 128 bytes into LDS (lane l lands at byte l*16 of the 1 KiB block):
// lane l serves row r = l>>3 of the block and physical 16-byte slot p = l&7, and fetches the logical chunk that the
// swizzle assigns to that slot (two lane offsets: blocks of 8 rows alternate in the swizzle's row bits).
// Wavefront w brings tile rows [32w, 32w + 32) with four such instructions.
// tile: uniform pointer to (first row of the tile, k step); row_block_bytes: 8 rows in bytes (uniform).
__device__ __forceinline__ void load_tile(const char* __restrict__ tile, uint32_t lane_off_even, uint32_t lane_off_odd,
                                          int64_t row_block_bytes, char* lds_tile, int wave) {
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    // scalar base + 32-bit lane offset: tell the compiler the base is uniform so the address stays in SGPRs
    const uint64_t u = reinterpret_cast<uint64_t>(tile + (wave * 4 + i) * row_block_bytes);
    const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)u);
    const uint32_t hi = __builtin_amdgcn_readfirstlane((uint32_t)(u >> 32));
    const char* src = reinterpret_cast<const char*>(((uint64_t)hi << 32) | lo);
    char* dst = lds_tile + (wave * 32 + i * 8) * kLmRowBytes;      // uniform
    __builtin_amdgcn_global_load_lds((const VRL_GLOBAL_AS void*)(src + ((i & 1) ? lane_off_odd : lane_off_even)), (VRL_LDS_AS void*)dst, 16, 0, 0);
  }
}

template <int DT>
__global__ __launch_bounds__(kLmWaves * 64, 1) void lmhead_partial_kernel(
    const uint16_t* __restrict__ W, const uint16_t* __restrict__ H, int64_t V, int64_t T, int64_t K, int64_t w_stride,
    int64_t h_stride, const float* __restrict__ temperature, int n_splits, int tiles_per_split,
    int xcd_map, float* __restrict__ partials) {
  extern __shared__ __attribute__((aligned(1024))) char lds[];  // [2 buffers][W tile, H tile]
  __shared__ float red[4][256][3];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);   // uniform: keeps tile addressing in scalar registers
  const int wv = wave >> 1;  // vocab quarter of the tile (8 wavefronts: 4 vocab quarters x 2 token halves)
  const int wt = wave & 1;   // token half of the tile
  // Workgroup -> (token block, split). Hardware deals workgroups round-robin over the 8 XCDs (id % 8); the 32 that
  // are resident on one XCD together should share operands through its L2: 8 token blocks x 4 splits per XCD
  // (each W slice read by 8 workgroups, each H slice by 4) when the grid has that shape, plain order otherwise.
  int split;
  int64_t tb;
  {
    const int64_t tblocks = (T + kLmTokens - 1) / kLmTokens;
    const int64_t id = blockIdx.x;
    if (xcd_map) {
      const int x = (int)(id & 7);
      const int64_t local = id >> 3;            // 0 .. tblocks*n_splits/8
      const int64_t tgroups = tblocks / 8;      // groups of 8 token blocks
      // super index over (tgroup, sgroup) pairs: 8 consecutive ones run at a time (one per XCD)
      const int64_t super = (local / 32) * 8 + x;
      const int64_t within = local % 32;
      const int64_t tg = super % tgroups;
      const int sg = (int)(super / tgroups);
      tb = tg * 8 + (within & 7);
      split = sg * 4 + (int)(within >> 3);
    } else {
      split = (int)(id % n_splits);
      tb = id / n_splits;
    }
  }
  const int64_t tok0 = tb * kLmTokens;
  const int64_t n_vtiles = (V + kLmVocab - 1) / kLmVocab;
  const int64_t vt_begin = (int64_t)split * tiles_per_split;
  int64_t vt_end = vt_begin + tiles_per_split;
  if (vt_end > n_vtiles) vt_end = n_vtiles;
  const int ksteps = (int)(K / kLmK);

  // per-lane softmax state for the 4 token columns this lane sees
  float m[4], s[4], t[4], c[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    m[j] = neg_inf();
    s[j] = 0.f;
    t[j] = 0.f;
    const int64_t tok = (tok0 + kLmTokens <= T ? tok0 : T - kLmTokens) + wt * 128 + j * 32 + (lane & 31);
    c[j] = make_scale<false>(temperature, tok).c;   // log2(e) / max(T, 1e-8), exactly what the finishing kernel uses
  }

  // fragment addressing: row (within its 32-row block) = lane&31, logical chunk = 2*sub + (lane>>5), sub in 0..3
  int phys[4];
#pragma unroll
  for (int sb = 0; sb < 4; ++sb) phys[sb] = (((2 * sb + (lane >> 5)) ^ ((lane >> 1) & 7)) * 16);
  const int fragoff_w = (wv * 64 + (lane & 31)) * kLmRowBytes;
  const int fragoff_h = kLmTileBytes + (wt * 128 + (lane & 31)) * kLmRowBytes;

  // Edge tiles are moved back so that all 256 rows exist (host guarantees V, T >= 256); the rows they share with
  // the tile before are masked in the epilogue (vocab) or not written (tokens).
  const int64_t tok0_ld = tok0 + kLmTokens <= T ? tok0 : T - kLmTokens;
  // physical 16-byte slot p of tile row R holds logical chunk p ^ ((R >> 1) & 7): 16 consecutive rows then cover
  // 16 distinct (row parity, slot) pairs, i.e. all 64 banks once per 16 lanes of a 128-bit read
  const int lr = lane >> 3;
  const int lc_e = (lane & 7) ^ (lr >> 1), lc_o = (lane & 7) ^ (4 + (lr >> 1));
  const uint32_t w_lane_e = (uint32_t)((lr * w_stride + lc_e * 8) * 2), w_lane_o = (uint32_t)((lr * w_stride + lc_o * 8) * 2);
  const uint32_t h_lane_e = (uint32_t)((lr * h_stride + lc_e * 8) * 2), h_lane_o = (uint32_t)((lr * h_stride + lc_o * 8) * 2);
  const int64_t w_blk = 8 * w_stride * 2, h_blk = 8 * h_stride * 2;
  const char* Wb = reinterpret_cast<const char*>(W);
  const char* Hb = reinterpret_cast<const char*>(H) + tok0_ld * h_stride * 2;

  // prefetch cursor: global step (tile, k step), two steps ahead of the compute cursor once the loop runs
  const int64_t total_steps = (vt_end > vt_begin ? (vt_end - vt_begin) : 0) * ksteps;
  int64_t pstep = 0, pvt = vt_begin;
  int pks = 0;
  // Loads of global step `pstep` into stage pstep & 1. Branch-free: past the last step the cursor stays on the last
  // step, whose tile is loaded once more into the stage nobody will read (in bounds, harmless), so the main loop is
  // one basic block.
  auto issue_always = [&]() {
    char* st = lds + (int)(pstep & 1) * 2 * kLmTileBytes;
    const int64_t vrow = (pvt + 1) * kLmVocab <= V ? pvt * kLmVocab : V - kLmVocab;
    load_tile(Wb + vrow * w_stride * 2 + (int64_t)pks * kLmRowBytes, w_lane_e, w_lane_o, w_blk, st, wave);
    load_tile(Hb + (int64_t)pks * kLmRowBytes, h_lane_e, h_lane_o, h_blk, st + kLmTileBytes, wave);
    const bool more = pstep + 1 < total_steps;
    ++pstep;
    const int nks = pks + 1;
    const bool wrap = nks == ksteps;
    pks = more ? (wrap ? 0 : nks) : pks;
    pvt = more ? (wrap ? pvt + 1 : pvt) : pvt;
  };
  typename LmFrag<DT>::type a[2][2], b[2][4];
  auto read_frags = [&](int set, const char* stage, int sb) {
#pragma unroll
    for (int i = 0; i < 2; ++i) a[set][i] = *reinterpret_cast<const typename LmFrag<DT>::type*>(stage + fragoff_w + i * 32 * kLmRowBytes + phys[sb]);
#pragma unroll
    for (int j = 0; j < 4; ++j) b[set][j] = *reinterpret_cast<const typename LmFrag<DT>::type*>(stage + fragoff_h + j * 32 * kLmRowBytes + phys[sb]);
  };
  if (total_steps > 0) {
    issue_always();   // step 0 -> stage 0
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    read_frags(0, lds, 0);
    issue_always();   // step 1 -> stage 1
  }

  int64_t step = 0;
  for (int64_t vt = vt_begin; vt < vt_end; ++vt) {
    lm_f32x16 acc[2][4];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

    for (int ks = 0; ks < ksteps; ++ks, ++step) {
      const char* cur = lds + (int)(step & 1) * 2 * kLmTileBytes;
      const char* nxt = lds + (int)((step + 1) & 1) * 2 * kLmTileBytes;
      // Quarter steps 0..2 compute from fragments and read the next quarter's fragments from `cur`.
#pragma unroll
      for (int sb = 0; sb < 3; ++sb) {
        const int cu = sb & 1, nx = cu ^ 1;
        read_frags(nx, cur, sb + 1);
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
          for (int j = 0; j < 4; ++j)
            acc[i][j] = LmFrag<DT>::mfma(a[cu][i], b[cu][j], acc[i][j]);
      }
      // The barrier sits BEFORE the last quarter's matrix instructions: its fragments (set 1) are in registers, so
      // every wavefront is done reading `cur`, and the next step's tile, requested a whole step ago, has landed in
      // `nxt`. Behind the barrier the next step's first fragments are fetched and the loads of the step after are
      // issued into `cur`, all underneath this quarter's matrix instructions.
      asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
      __syncthreads();
      read_frags(0, nxt, 0);
      issue_always();
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
          acc[i][j] = LmFrag<DT>::mfma(a[1][i], b[1][j], acc[i][j]);
    }

    // epilogue of this vocab tile: fold 64 logits per token column into the running state (two passes over the
    // accumulators: maximum, then exponentials; nothing is buffered)
    const bool edge = (vt + 1) * kLmVocab > V;
    const int64_t vrow0 = (edge ? V - kLmVocab : vt * kLmVocab) + wv * 64 + 4 * (lane >> 5);
    const int64_t vfirst = vt * kLmVocab;   // rows below belong to the tile before
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      float bm = neg_inf();
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        // one 32x32 block (16 accumulator registers) at a time; the scheduling barrier keeps the compiler from
        // pulling the next blocks' accumulator copies forward, which would spill registers across the main loop
        float x[16];
#pragma unroll
        for (int v = 0; v < 16; ++v) x[v] = acc[i][j][v];
        if (edge) {
#pragma unroll
          for (int v = 0; v < 16; ++v) {
            const int64_t vr = vrow0 + i * 32 + 8 * (v >> 2) + (v & 3);
            x[v] = vr >= vfirst ? x[v] : neg_inf();
          }
        }
#pragma unroll
        for (int v = 0; v < 16; ++v) bm = __builtin_fmaxf(bm, x[v]);
        __builtin_amdgcn_sched_barrier(0);
      }
      bm *= c[j];   // c > 0: the maximum commutes with the scale
      if (bm > m[j]) {
        const float al = hw_exp2(m[j] - bm);  // m = -inf -> 0
        const float dm = (m[j] == neg_inf()) ? 0.f : (m[j] - bm);
        t[j] = al * (t[j] + dm * s[j]);
        s[j] = al * s[j];
        m[j] = bm;
      }
      const float sub = (m[j] == neg_inf()) ? 0.f : m[j];
      float ps = 0.f, pt = 0.f;
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        float x[16];
#pragma unroll
        for (int v = 0; v < 16; ++v) x[v] = acc[i][j][v];
        if (edge) {
#pragma unroll
          for (int v = 0; v < 16; ++v) {
            const int64_t vr = vrow0 + i * 32 + 8 * (v >> 2) + (v & 3);
            x[v] = vr >= vfirst ? x[v] : neg_inf();
          }
        }
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          const float d = __builtin_fmaf(x[v], c[j], -sub);
          const float e = hw_exp2(d);
          ps += e;
          pt = __builtin_fmaf(e, (e == 0.f) ? 0.f : d, pt);
        }
        __builtin_amdgcn_sched_barrier(0);
      }
      s[j] += ps;
      t[j] += pt;
    }
  }

  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // the last, redundant loads still target the LDS stages
  // combine: lanes l and l^32 hold the same tokens (other vocab rows), then the two vocab-half waves via LDS
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const float om = __shfl_xor(m[j], 32);
    const float os = __shfl_xor(s[j], 32);
    const float ot = __shfl_xor(t[j], 32);
    const float M = __builtin_fmaxf(m[j], om);
    float S = 0.f, Tt = 0.f;
    if (M != neg_inf()) {
      const float a1 = hw_exp2(m[j] - M), a2 = hw_exp2(om - M);
      const float d1 = (m[j] == neg_inf()) ? 0.f : m[j] - M;
      const float d2 = (om == neg_inf()) ? 0.f : om - M;
      S = a1 * s[j] + a2 * os;
      Tt = a1 * (t[j] + d1 * s[j]) + a2 * (ot + d2 * os);
    }
    if (lane < 32) {
      const int col = wt * 128 + j * 32 + lane;
      red[wv][col][0] = M;
      red[wv][col][1] = S;
      red[wv][col][2] = Tt;
    }
  }
  __syncthreads();
  if (tid < 256) {
    const int col = tid;  // 256 token columns
    const int64_t tok = tok0_ld + col;
    if (tok >= tok0) {
      float M = red[0][col][0];
#pragma unroll
      for (int q = 1; q < 4; ++q) M = __builtin_fmaxf(M, red[q][col][0]);
      float S = 0.f, Tt = 0.f;
      if (M != neg_inf()) {
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const float mq = red[q][col][0];
          const float aq = hw_exp2(mq - M);
          const float dq = (mq == neg_inf()) ? 0.f : mq - M;
          S += aq * red[q][col][1];
          Tt += aq * (red[q][col][2] + dq * red[q][col][1]);
        }
      }
      float* p = partials + (tok * n_splits + split) * 4;
      p[0] = M;
      p[1] = S;
      p[2] = Tt;
      p[3] = 0.f;
    }
  }
}


// grid.x = ceil(T / 4), block = 256: wavefront w of a workgroup finishes token blockIdx.x * 4 + w.
template <int DT>
__global__ __launch_bounds__(256) void lmhead_finish_kernel(
    const char* __restrict__ W, const char* __restrict__ H, int64_t V, int64_t T, int64_t K, int64_t w_stride,
    int64_t h_stride, const int64_t* __restrict__ labels, const float* __restrict__ temperature, int n_splits,
    const float* __restrict__ partials, float* __restrict__ out_logprob, float* __restrict__ out_entropy,
    float* __restrict__ out_lse, int32_t* err_flag) {
  using E = Elem<DT>;
  const int lane = threadIdx.x & 63;
  const int64_t tok = static_cast<int64_t>(blockIdx.x) * 4 + (threadIdx.x >> 6);
  if (tok >= T) return;  // the whole wavefront leaves; this kernel has no barrier
  float xl = 0.f;
  bool label_ok = true;
  if (out_logprob != nullptr) {
    const int64_t label = labels[tok];
    label_ok = label >= 0 && label < V;
    if (label_ok) {
      const u32x4* hp = reinterpret_cast<const u32x4*>(H + tok * h_stride * 2);
      const u32x4* wp = reinterpret_cast<const u32x4*>(W + label * w_stride * 2);
      float acc = 0.f;
      for (int64_t k = lane; k < K / 8; k += 64) {
        float hv[8], wv[8];
        E::unpack(hp[k], hv);
        E::unpack(wp[k], wv);
#pragma unroll
        for (int i = 0; i < 8; ++i) acc = __builtin_fmaf(hv[i], wv[i], acc);
      }
      xl = wave_sum(acc);
    }
  }
  Part p;
  p.m = neg_inf();
  p.s = 0.f;
  p.t = 0.f;
  p.q = 0.f;
  if (lane < n_splits) {
    const float* src = partials + (tok * n_splits + lane) * 4;
    p.m = src[0];
    p.s = src[1];
    p.t = src[2];
  }
  const float M = wave_max(p.m);
  rescale(p, M);
  Part w;
  w.m = M;
  w.s = wave_sum(p.s);
  w.t = wave_sum(p.t);
  w.q = 0.f;
  if (lane == 0) {
    const Scale<false> sc = make_scale<false>(temperature, tok);
    finalize_row<false, false>(w, xl, label_ok, sc, tok, out_logprob, out_entropy, nullptr, out_lse, err_flag);
  }
}

}  // namespace vrl
